// Token-stationary fused SwiGLU feed-forward with FP8 (OCP e4m3fn, per-tensor scales) MFMA operands for gfx950:
//   h   = norm_weight ? bf16(rmsnorm(x, norm_weight)) : x                      quantised with scale amax_x / 448
//   g,u = chunk2( (q(h) q(w_up)^T) * s_x * s_up + b_up )                       fp32
//   hid = silu(g) * u   (fp32, not rounded to bf16 in between)                 quantised with scale amax_hidden / 448
//   out = bf16( (q(hid) q(w_down)^T) * s_hid * s_down + b_down + residual )    one rounding
// which is the chain of two per-tensor-scaled dense layers (quantize -> matmul -> dequantize, SiLU-gate epilogue on the
// first, residual epilogue on the second) with the [M, F] hidden state never written to memory.
//
// A per-tensor scale of the hidden state needs its maximum over ALL tokens before any of it can be quantised, so the
// layer is two launches of one scheme:
//   pass 1  up projection + SiLU-gate only; the result is reduced to max |hid| (one atomic per workgroup) and dropped;
//   pass 2  up projection again, SiLU-gate, quantisation with the now known scale, down projection, epilogue.
// Recomputing the up projection (2/3 of the layer's products) costs less than writing the hidden state in 16 bits and
// reading it back (2 * M * F * 2 bytes), and far less at the valid-token counts of a padded batch.
//
// Scheme: a wavefront owns 32 tokens (pass 1: 64) for the whole kernel and keeps their quantised rows as MFMA B operands
// of v_mfma_scale_f32_32x32x64_f8f6f4 (lane (l32, hh) holds the 32 bytes k = 64 ks + 32 hh .. + 31 of token l32); the
// weights stream L2 -> LDS by DMA in fragment order (2 KB fragments = 32 rows x 64 k, written as two 1 KB halves) through
// two buffers, one barrier per 32 hidden units.
// A chunk of 64 hidden units is four sub-chunks of 16: the up fragment of a sub-chunk stacks 16 gated rows on their 16
// partner rows, so one accumulator holds g (registers 0..7) and u (8..15) of eight hidden units of the lane's token;
// silu(g) * u of the four sub-chunks are the lane's 32 bytes of the down projection's B operand (the k order of the
// packed W_down fragments follows that register order). The down projection of a chunk is issued one chunk late, behind
// the sub-chunks of the next one (the blob stores the down fragments of chunk c - 1 next to the up fragments of chunk c).
// Workgroups are small (4 wavefronts, 58 KB of LDS) so that two of them share a compute unit: the token loads, the
// normalisation and the output stores of one overlap with the matrix work of the other, and the bursts of HBM traffic at
// the start and the end of a tile spread out.
#include <cstdlib>

#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kF8Frag = 2048;     // bytes of one 32 x 64 e4m3 fragment
constexpr int kF8Chunk = 64;      // hidden units per chunk (one k-step of the down projection)
constexpr int kF8ScaleOne = 127;  // E8M0 exponent of 1.0 (unit block scales)

struct FfnFp8Params {
  const bf16_t* x;            // [M, D] row stride ldx
  const bf16_t* norm_w;       // [D] or null
  const uint8_t* packed;      // blob of taac_ffn_fp8_pack_weights
  const bf16_t* b_up;         // [2F] or null
  const bf16_t* b_down;       // [D] or null
  const bf16_t* residual;     // [M, D] row stride ldr or null
  bf16_t* out;                // [M, D] row stride ldo
  const bf16_t* next_norm_w;  // [D] or null: norm weight of the layer that consumes out (for amax_next)
  const float* amax_x;
  const float* amax_up;
  const float* amax_down;
  float* amax_hidden;         // written by pass 1 (atomic max), read by pass 2
  float* amax_next;           // atomic max of |bf16(rmsnorm(out, next_norm_w))| (or of |out|), or null
  int64_t M, ldx, ldr, ldo;
  int32_t F;
  int32_t gate_first;
  float eps, next_eps;
  const int32_t* rows;
  const int32_t* n_rows;
};

// Hidden unit (0..15) of row slot m16 of the gated (or partner) half of an up fragment: accumulator register j < 8 of
// lane half hh then holds unit 8 * hh + j.
__host__ __device__ __forceinline__ int f8_unit_of_slot(int m16) {
  return 8 * ((m16 >> 2) & 1) + 4 * (m16 >> 3) + (m16 & 3);
}

__device__ __forceinline__ float f8_clamp(float x) { return __builtin_fminf(__builtin_fmaxf(x, -448.f), 448.f); }

// Two floats -> two e4m3 bytes in the low (hi = false) or high half of `old`.
template <bool HI>
__device__ __forceinline__ int f8_pack2(float a, float b, int old) {
  return __builtin_amdgcn_cvt_pk_fp8_f32(f8_clamp(a), f8_clamp(b), old, HI);
}

template <int OFFSET>
__device__ __forceinline__ void f8_lds_read16(u32x4& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}
template <int N>
__device__ __forceinline__ void f8_lds_wait(u32x4& a, u32x4& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

__device__ __forceinline__ float f8_pair_sum(float v) {  // v + the value of lane ^ 32
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, static_cast<uint32_t>(r[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(r[1]));
}

// Maximum over the workgroup, then one atomic max on the float's bit pattern (non-negative floats order like their
// bits); skipped when the global value already covers it. `red` holds one float per wavefront.
__device__ __forceinline__ void f8_block_atomic_max(float m, float* dst, float* red, int wave, int lane, int nwaves) {
  m = group_max<kWave>(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  if (wave == 0 && lane == 0) {
    for (int w = 1; w < nwaves; ++w) m = fmaxf(m, red[w]);
    if (m > __builtin_nontemporal_load(dst)) atomicMax(reinterpret_cast<unsigned int*>(dst), __float_as_uint(m));
  }
}

// ---- weight packing -------------------------------------------------------------------------------------------------
// Blob = 2 * F / 64 steps of 32 hidden units, then a tail. Step h covers sub-chunks s = 2 (h % 2), 2 (h % 2) + 1 of
// chunk c = h / 2 (hidden units 64 c .. 64 c + 63); per sub-chunk it holds the D / 64 up fragments (k-step ks) of
// (c, s) followed by the D / 128 down fragments (row blocks s * D / 128 ..) of chunk c - 1 (cyclically: chunk F / 64 - 1
// for c = 0, where they meet a zero operand). The tail holds the D / 32 down fragments of the last chunk.
// A fragment is the LDS image: half h (1 KB) holds for lane l the 16 bytes k = 32 * (l / 32) + 16 h .. + 15 of row l % 32.
//   up fragment:   row slot m = l % 32: weight row [(m < 16) == gate_first ? 0 : F] + 64 c + 16 s + unit(m % 16), columns
//                  64 ks + k;
//   down fragment: row mb * 32 + l % 32; k index kk = 32 hh + 8 s + j is hidden unit 64 c + 16 s + 8 hh + j.
// Values are quantised as q = sat(w / (amax / 448)) with a true division (bit-identical to taac_quantize_fp8).
__device__ __forceinline__ uint32_t f8_quant4(const bf16_t* v, float scale) {
  float f[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) f[e] = f8_clamp(static_cast<float>(v[e]) / scale);
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
  return static_cast<uint32_t>(w);
}

__device__ __forceinline__ void ffn_fp8_pack_piece(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                                   const float* __restrict__ amax_up, const float* __restrict__ amax_down,
                                                   u32x4* __restrict__ packed, int D, int F, int gate_first, int64_t gid) {
  const int KS = D / 64, MB = D / 32, DPS = MB / 4, SUBF = KS + DPS, NC = F / kF8Chunk;
  const int64_t stream_frags = static_cast<int64_t>(NC) * 4 * SUBF;
  const int64_t total = (stream_frags + MB) * 128;  // 16-byte pieces
  if (gid >= total) return;
  const int lane = static_cast<int>(gid % 64);
  const int half = static_cast<int>((gid / 64) % 2);
  const int64_t fi = gid / 128;
  const int l32 = lane % 32, hh = lane / 32;
  bool up = false;
  int64_t chunk;
  int sub = 0, ks = 0, mb = 0;
  if (fi < stream_frags) {
    const int64_t sidx = fi / SUBF;  // sub-chunk counter over the whole stream
    const int rr = static_cast<int>(fi % SUBF);
    sub = static_cast<int>(sidx % 4);
    chunk = sidx / 4;
    if (rr < KS) {
      up = true;
      ks = rr;
    } else {
      mb = sub * DPS + rr - KS;
      chunk = (chunk + NC - 1) % NC;
    }
  } else {
    mb = static_cast<int>(fi - stream_frags);
    chunk = NC - 1;
  }
  bf16_t v[16];
  float scale;
  if (up) {
    const int64_t row = ((l32 < 16) == (gate_first != 0) ? 0 : F) + chunk * kF8Chunk + 16 * sub + f8_unit_of_slot(l32 & 15);
    const bf16_t* src = w_up + row * D + ks * 64 + hh * 32 + half * 16;
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = src[e];
    scale = fmaxf(*amax_up, 1e-12f) / 448.0f;
  } else {
    const bf16_t* src = w_down + static_cast<int64_t>(mb * 32 + l32) * F + chunk * kF8Chunk;
#pragma unroll
    for (int b = 0; b < 16; ++b) v[b] = src[16 * (2 * half + b / 8) + 8 * hh + b % 8];
    scale = fmaxf(*amax_down, 1e-12f) / 448.0f;
  }
  const u32x4 q = {f8_quant4(v, scale), f8_quant4(v + 4, scale), f8_quant4(v + 8, scale), f8_quant4(v + 12, scale)};
  packed[gid] = q;
}

__global__ __launch_bounds__(256) void ffn_fp8_pack_kernel(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                                           const float* __restrict__ amax_up,
                                                           const float* __restrict__ amax_down, u32x4* __restrict__ packed,
                                                           int D, int F, int gate_first) {
  ffn_fp8_pack_piece(w_up, w_down, amax_up, amax_down, packed, D, F, gate_first,
                     static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x);
}

// ---- shared pieces ----------------------------------------------------------------------------------------------------
__device__ __forceinline__ int64_t f8_token_count(const FfnFp8Params& p) {
  if (p.rows == nullptr) return p.M;
  const int64_t n = *p.n_rows;
  return n < p.M ? n : p.M;
}
__device__ __forceinline__ int64_t f8_token_row(const FfnFp8Params& p, int64_t count, int64_t tok) {
  tok = tok < count ? tok : count - 1;
  return p.rows != nullptr ? static_cast<int64_t>(p.rows[tok]) : tok;
}

// Loads the 32 token rows of one tile, optionally RMS-normalises them (rounded to bf16 as the stand-alone norm rounds its
// output) and quantises them into B-operand fragments: xq[ks] = bytes k = 64 ks + 32 hh .. + 31 of token l32.
template <int D>
__device__ __forceinline__ void f8_load_tokens(const FfnFp8Params& p, int64_t row, const bf16_t* norm_w_lds, float inv_scale,
                                               int hh, i32x8 (&xq)[D / 64]) {
  constexpr int KS = D / 64;
  const bf16_t* src = p.x + row * p.ldx + hh * 32;
  bf16x8 raw[KS][4];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
#pragma unroll
    for (int c = 0; c < 4; ++c) raw[ks][c] = *reinterpret_cast<const bf16x8*>(src + ks * 64 + c * 8);
  float scale = 1.0f;
  if (p.norm_w != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float v = static_cast<float>(raw[ks][c][e]);
          ss = fmaf(v, v, ss);
        }
    scale = rsqrtf(f8_pair_sum(ss) * (1.0f / D) + p.eps);
  }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    int q[8];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float f[8];
      if (p.norm_w != nullptr) {
        const bf16x8 wv = *reinterpret_cast<const bf16x8*>(norm_w_lds + ks * 64 + hh * 32 + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          f[e] = static_cast<float>(static_cast<bf16_t>(static_cast<float>(raw[ks][c][e]) * scale * static_cast<float>(wv[e])));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = static_cast<float>(raw[ks][c][e]);
      }
      int lo = f8_pack2<false>(f[0] * inv_scale, f[1] * inv_scale, 0);
      lo = f8_pack2<true>(f[2] * inv_scale, f[3] * inv_scale, lo);
      int hi = f8_pack2<false>(f[4] * inv_scale, f[5] * inv_scale, 0);
      hi = f8_pack2<true>(f[6] * inv_scale, f[7] * inv_scale, hi);
      q[2 * c] = lo;
      q[2 * c + 1] = hi;
    }
    xq[ks] = i32x8{q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7]};
    asm volatile("" : "+v"(xq[ks]));
  }
}

// Up-projection bias as the A operand of one bf16 MFMA per sub-chunk: entry (chunk * 4 + s) * 32 + m belongs to row slot
// m of sub-chunk s (slots 0..15 the gated units, 16..31 their partners) and holds bias / dq as a (high, low) pair of bf16
// values (k = 0 and k = 1 of the fragment; the B operand is 1 at both), so that the product adds bias / dq to the
// accumulator with ~16 bits of mantissa. dq is the dequantisation factor of the up projection: the accumulators then hold
// (projection + bias) / dq and the activation works on them without a per-element bias or scale operation.
__device__ __forceinline__ void f8_stage_up_bias(const bf16_t* b_up, uint32_t* dst, int F, int gate_first, float inv_dq, int tid,
                                                 int nthreads) {
  for (int i = tid; i < 2 * F; i += nthreads) {
    const int sub = i / 32, m = i % 32;
    const int src = ((m < 16) == (gate_first != 0) ? 0 : F) + sub * 16 + f8_unit_of_slot(m % 16);
    const float v = static_cast<float>(b_up[src]) * inv_dq;
    const bf16_t hi = static_cast<bf16_t>(v);
    const bf16_t lo = static_cast<bf16_t>(v - static_cast<float>(hi));
    dst[i] = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, hi)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, lo)) << 16);
  }
}

// ---- the kernel -------------------------------------------------------------------------------------------------------
// PASS2 = false: up projection + activation, max |hid| -> amax_hidden.   PASS2 = true: the whole layer.
// A wavefront owns TT tiles of 32 tokens; every weight fragment read from LDS feeds TT MFMAs. NW wavefronts per workgroup.
// BIAS: an up-projection bias is present. The activation works on the raw accumulators a = (projection + bias) / dq:
//   silu(g) * u = a_g * a_u * dq^2 / (1 + exp2(-log2(e) * dq * a_g)),
// the constant factors are applied once (to the maximum in pass 1, folded into the quantisation factor in pass 2).
// Software pipeline inside a wavefront: two accumulator sets; while the MFMAs of sub-chunk s are issued into one set, the
// activation of sub-chunk s - 1 is evaluated from the other, a few values behind every MFMA, so that the vector ALU works
// under the matrix unit. The down projection of a chunk follows one chunk late (its B operand, the quantised hidden state
// of the previous chunk, is complete once the first sub-chunk of the current chunk has been issued).
// LDS: [2 weight buffers][b_down (D) | norm weight (D) | next norm weight (D)][16 floats][BIAS: bias pairs (2F dwords)]
template <int D, int TT, int NW, bool PASS2, bool BIAS>
__global__ __launch_bounds__(NW* kWave, 2) void swiglu_ffn_fp8_kernel(const FfnFp8Params p) {
  constexpr int KS = D / 64;                    // k-steps of the up projection = up fragments per sub-chunk
  constexpr int MB = D / 32;                    // row blocks of the down projection
  constexpr int DPS = MB / 4;                   // down fragments behind every sub-chunk
  constexpr int SUBF = KS + DPS;                // fragments per sub-chunk in the blob
  constexpr int CSUB = KS + (PASS2 ? DPS : 0);  // fragments per sub-chunk this pass stages and consumes
  constexpr int STEPF = 2 * CSUB;               // fragments per step (two sub-chunks)
  constexpr int kBuf = STEPF * kF8Frag;
  constexpr int DPW = STEPF * 2 / NW;           // 1 KB DMA instructions per wavefront and step
  static_assert(STEPF * 2 % NW == 0 && (MB * 2) % NW == 0, "the transfers of a step divide over the wavefronts");
  constexpr int P = 3;                          // fragments in flight (a fourth makes the register allocation spill)
  constexpr int EPM = 8 / KS;                   // activation values evaluated behind every up MFMA (2 or 4)
  constexpr int kTokPerWg = NW * 32 * TT;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int F = p.F;
  bf16_t* bdown_lds = reinterpret_cast<bf16_t*>(smem + 2 * kBuf);
  bf16_t* normw_lds = bdown_lds + D;
  bf16_t* nextw_lds = normw_lds + D;
  float* red = reinterpret_cast<float*>(nextw_lds + D);
  uint32_t* bias_lds = reinterpret_cast<uint32_t*>(red + 16);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int64_t count = f8_token_count(p);
  const int64_t wg_tok0 = static_cast<int64_t>(blockIdx.x) * kTokPerWg;
  if (wg_tok0 >= count) return;  // whole workgroup
  const int64_t tok0 = wg_tok0 + wave * (32 * TT);
  const bool active = tok0 < count;  // a wavefront beyond the tokens only helps staging

  // Step h of the weight stream -> buffer buf. Pass 2 takes the step as it lies in the blob; pass 1 only its up fragments.
  const int nsteps = 2 * (F / kF8Chunk);
  auto stage = [&](int h, int buf) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
    const uint8_t* step_src = p.packed + static_cast<int64_t>(h) * (2 * SUBF * kF8Frag);
    uint8_t* dst = smem + buf * kBuf + wave * (DPW * 1024);
#pragma unroll
    for (int i = 0; i < DPW; ++i) {
      const int j = wave * DPW + i;           // transfer j of the step: half j % 2 of staged fragment j / 2
      const int f = j / 2, q = f / CSUB, rr = f % CSUB;
      lds_dma16_offset(step_src + ((q * SUBF + rr) * 2 + j % 2) * 1024, lane_off, dst + i * 1024);
    }
  };
  // The down fragments of the last chunk (the tail of the blob) -> buffer buf, fragment mb at index mb.
  [[maybe_unused]] auto stage_tail = [&](int buf) {
    constexpr int TPW = MB * 2 / NW;
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
    const uint8_t* src = p.packed + static_cast<int64_t>(nsteps) * (2 * SUBF * kF8Frag) + wave * (TPW * 1024);
    uint8_t* dst = smem + buf * kBuf + wave * (TPW * 1024);
#pragma unroll
    for (int i = 0; i < TPW; ++i) lds_dma16_offset(src + i * 1024, lane_off, dst + i * 1024);
  };

  stage(0, 0);
  const float amax_x = fmaxf(*p.amax_x, 1e-12f);
  const float amax_up = fmaxf(*p.amax_up, 1e-12f);
  const float dq1 = (amax_x / 448.0f) * (amax_up / 448.0f);
  if (BIAS) f8_stage_up_bias(p.b_up, bias_lds, F, p.gate_first, 1.0f / dq1, tid, NW * kWave);
  stage_bias(p.b_down, bdown_lds, D, tid, NW * kWave);
  stage_bias(p.norm_w, normw_lds, D, tid, NW * kWave);
  stage_bias(p.next_norm_w, nextw_lds, D, tid, NW * kWave);

  const float exp_scale = -1.4426950408889634f * dq1;  // exp2(exp_scale * a_g) = exp(-g)
  float quant_scale = 1.f, dq2 = 0.f;                  // pass 2: a_g a_u sigmoid -> units of the hidden state's e4m3 grid
  if (PASS2) {
    const float amax_h = fmaxf(*p.amax_hidden, 1e-12f);
    quant_scale = dq1 * dq1 * (448.0f / amax_h);
    dq2 = (amax_h / 448.0f) * (fmaxf(*p.amax_down, 1e-12f) / 448.0f);
  }
  vm_wait<0>();
  __syncthreads();  // biases and norm weights are in LDS, chunk 0 has landed

  i32x8 xq[TT][KS];
  if (active) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
      f8_load_tokens<D>(p, f8_token_row(p, count, tok0 + t * 32 + l32), normw_lds, 448.0f / amax_x, hh, xq[t]);
  }

  f32x16 oacc[PASS2 ? TT : 1][PASS2 ? MB : 1];
  if (PASS2) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[t][mb][j] = 0.f;
  }
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // pass 1: running exact maximum in accumulator units (dq^2 taken out), seeded with the published value (a hair below it,
  // so that rounding in the conversion cannot hide a value that is above everything evaluated so far)
  float hmax = PASS2 ? 0.f : __builtin_nontemporal_load(p.amax_hidden) / (dq1 * dq1) * (1.0f - 1e-6f);
  // hb_cur: the quantised hidden state of the previous chunk (B operand of its pending down projection; its last two
  // dwords arrive during the first sub-chunk of the current chunk); hb_nxt: the one being assembled. Before the first
  // chunk both are zero, and the zero hb_cur multiplies chunk 0's own (finite) down fragments.
  int hb_cur[TT][8], hb_nxt[TT][8];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int i = 0; i < 8; ++i) hb_cur[t][i] = hb_nxt[t][i] = 0;
  f32x16 gu[2][TT];  // set s % 2 receives sub-chunk s; zero accumulators give a zero activation before the first one
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int t = 0; t < TT; ++t) gu[a][t] = zero16;

  const uint32_t smem_off = lds_offset(smem) + lane * 16;
  // B operand of the bias product: 1 at k = 0 and k = 1 (both live in the lower half-wavefront)
  u32x4 ones_bits = {hh == 0 ? 0x3f803f80u : 0u, 0u, 0u, 0u};
  asm volatile("" : "+v"(ones_bits));
  const bf16x8 ones = __builtin_bit_cast(bf16x8, ones_bits);

  // a_g * a_u * q / (1 + exp(-g)) of hidden unit j of the lane (accumulator registers j and 8 + j); the factor q (pass 2:
  // the quantisation factor, pass 1: 1) is folded into the denominator: q / (1 + e) = 1 / ((1 + e) / q).
  const float inv_q = 1.0f / quant_scale;
  auto activate = [&](const f32x16& acc, int j) -> float {
    const float e = __builtin_amdgcn_exp2f(acc[j] * exp_scale);
    return (acc[j] * acc[8 + j]) * __builtin_amdgcn_rcpf(fmaf(e, inv_q, inv_q));
  };
  // Values r * EPM .. + EPM - 1 of the sub-chunk held in `acc`: reduced into hmax (pass 1) or quantised into the B operand
  // dwords 2 * ps, 2 * ps + 1 of `hb` (pass 2; value j is byte 8 * ps + j of the lane's 32).
  // Pass 1 only needs max |a_g a_u sigmoid(g)|. As sigmoid < 1, |a_g a_u| bounds it: the pieces collect that bound (a
  // multiply and half a maximum per value), and the exact values of a sub-chunk are evaluated only when some lane's bound
  // exceeds its running exact maximum (checked once per sub-chunk, wavefront-uniform). The running maximum starts from what
  // earlier workgroups have already published in amax_hidden, so after the first round of workgroups almost every
  // sub-chunk takes the cheap route; skipped values are below a value that was evaluated exactly, so the result is exact.
  float bound = 0.f;
  auto bound_piece = [&](const f32x16& acc, auto rc) {
    constexpr int r = decltype(rc)::value;
#pragma unroll
    for (int e = 0; e < EPM; ++e) bound = fmaxf(bound, fabsf(acc[r * EPM + e] * acc[8 + r * EPM + e]));
  };
  auto exact_subchunk = [&](const f32x16 (&acc)[TT]) {
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j) hmax = fmaxf(hmax, fabsf(activate(acc[t], j)));
  };
  auto activation_piece = [&](const f32x16& acc, int (&hb)[8], auto psc, auto rc) {
    constexpr int ps = decltype(psc)::value, r = decltype(rc)::value;
    if constexpr (!PASS2) {
      bound_piece(acc, rc);
      return;
    }
    float h[EPM];
#pragma unroll
    for (int e = 0; e < EPM; ++e) h[e] = activate(acc, r * EPM + e);
    if constexpr (!PASS2) {
      static_assert(true, "pass 1 does not come here");
    } else if constexpr (EPM == 2) {
      if constexpr (r % 2 == 0)
        hb[2 * ps + r / 2] = f8_pack2<false>(h[0], h[1], 0);
      else
        hb[2 * ps + r / 2] = f8_pack2<true>(h[0], h[1], hb[2 * ps + r / 2]);
    } else {
      const int w = f8_pack2<false>(h[0], h[1], 0);
      hb[2 * ps + r] = f8_pack2<true>(h[2], h[3], w);
    }
  };

  // One step = two sub-chunks: its fragments are consumed in their LDS order, per sub-chunk KS up fragments then (pass 2)
  // DPS down fragments of the previous chunk, each fragment feeding TT MFMAs. `half` selects sub-chunks 0, 1 or 2, 3.
  auto run_step = [&](const uint32_t wb, auto halfc, const uint32_t (&brow)[4]) {
    constexpr int half = decltype(halfc)::value;
    u32x4 rlo[P], rhi[P];
    auto read_stream = [&](auto ic, int slot) {
      constexpr int i = decltype(ic)::value;
      f8_lds_read16<i * kF8Frag>(rlo[slot], wb);
      f8_lds_read16<i * kF8Frag + 1024>(rhi[slot], wb);
    };
    static_for<P>([&](auto ic) { read_stream(ic, decltype(ic)::value); });
    static_for<STEPF>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int s = 2 * half + i / CSUB, r = i % CSUB;
      constexpr int after = 2 * (P - 1 < STEPF - 1 - i ? P - 1 : STEPF - 1 - i);
      f8_lds_wait<after>(rlo[i % P], rhi[i % P]);
      const u32x4 lo = rlo[i % P], hi = rhi[i % P];
      const i32x8 wf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      if constexpr (r < KS) {
        // ---- up projection of sub-chunk s into set s % 2; behind every MFMA a piece of the activation of sub-chunk
        // s - 1 (the other set). For s = 0 that is sub-chunk 3 of the previous chunk, which completes hb_cur. ------------
        constexpr int a = s % 2, pa = (s + 1) % 2, ps = (s + 3) % 4;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          gu[a][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, xq[t][r], r == 0 ? zero16 : gu[a][t], 0, 0, 0,
                                                                       kF8ScaleOne, 0, kF8ScaleOne);
          if constexpr (BIAS && r == KS - 1) {
            // the bias product closes the chain: its result is not needed before the next sub-chunk, whereas in front of
            // the chain the first product would have to wait for it
            const u32x4 bias_bits = {brow[s], 0u, 0u, 0u};
            gu[a][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bias_bits), ones, gu[a][t], 0, 0, 0);
          }
          asm volatile("" : "+v"(gu[a][t]));
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (s == 0)
            activation_piece(gu[pa][t], hb_cur[t], std::integral_constant<int, ps>{}, std::integral_constant<int, r>{});
          else
            activation_piece(gu[pa][t], hb_nxt[t], std::integral_constant<int, ps>{}, std::integral_constant<int, r>{});
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (!PASS2 && r == KS - 1) {
          // sub-chunk s - 1 (set pa) has been bounded; its accumulators are overwritten by sub-chunk s + 1
          if (__builtin_amdgcn_ballot_w64(bound > hmax) != 0) exact_subchunk(gu[pa]);
          bound = 0.f;
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        // ---- down projection of the previous chunk, row block s * DPS + r - KS ------------------------------------------
        constexpr int mb = s * DPS + r - KS;
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const i32x8 hb = {hb_cur[t][0], hb_cur[t][1], hb_cur[t][2], hb_cur[t][3],
                            hb_cur[t][4], hb_cur[t][5], hb_cur[t][6], hb_cur[t][7]};
          oacc[PASS2 ? t : 0][PASS2 ? mb : 0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              wf, hb, oacc[PASS2 ? t : 0][PASS2 ? mb : 0], 0, 0, 0, kF8ScaleOne, 0, kF8ScaleOne);
          asm volatile("" : "+v"(oacc[PASS2 ? t : 0][PASS2 ? mb : 0]));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (i + P < STEPF) read_stream(std::integral_constant<int, i + P>{}, i % P);
    });
  };

  const int nchunks = nsteps / 2;
  for (int c = 0; c < nchunks; ++c) {
    // bias fragments of the chunk's four sub-chunks: one dword per lane (row slot l32), k = 0, 1 of the lower half-wavefront
    uint32_t brow[4] = {0u, 0u, 0u, 0u};
    if (BIAS && active) {
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const uint32_t w = bias_lds[(c * 4 + s4) * 32 + l32];
        brow[s4] = hh == 0 ? w : 0u;
      }
    }
    if (!PASS2) hmax = group_max<kWave>(hmax);  // share the running maximum inside the wavefront once per chunk
    // first half: buffer 0
    stage(2 * c + 1, 1);
    if (active) run_step(smem_off, std::integral_constant<int, 0>{}, brow);
    vm_wait<0>();  // the next step's weights (the only vector-memory operations of the loop)
    __syncthreads();
    // second half: buffer 1; the step after it (or, after the last one, the pending down fragments) goes to buffer 0
    if (c + 1 < nchunks)
      stage(2 * c + 2, 0);
    else if (PASS2)
      stage_tail(0);
    if (active) {
      run_step(smem_off + kBuf, std::integral_constant<int, 1>{}, brow);
      if (PASS2) {  // dwords 0..5 of the chunk just processed; 6, 7 follow during the next chunk's first sub-chunk
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int i = 0; i < 6; ++i) hb_cur[t][i] = hb_nxt[t][i];
      }
    }
    vm_wait<0>();
    __syncthreads();
  }

  // the last sub-chunk's activation is still pending (accumulator set 1)
  if (active) {
    if constexpr (PASS2) {
#pragma unroll
      for (int t = 0; t < TT; ++t)
        static_for<KS>([&](auto rc) { activation_piece(gu[1][t], hb_cur[t], std::integral_constant<int, 3>{}, rc); });
    } else {
      exact_subchunk(gu[1]);
    }
  }
  if constexpr (!PASS2) {
    f8_block_atomic_max(active ? hmax * (dq1 * dq1) : 0.f, p.amax_hidden, red, wave, lane, NW);
    return;
  } else {
    // ---- the down projection of the last chunk is still pending; its fragments were staged into buffer 0 ---------------
    float nmax = 0.f;
    if (active) {
      u32x4 tlo[MB], thi[MB];
      static_for<MB>([&](auto ic) {
        constexpr int mb = decltype(ic)::value;
        f8_lds_read16<mb * kF8Frag>(tlo[mb], smem_off);
        f8_lds_read16<mb * kF8Frag + 1024>(thi[mb], smem_off);
      });
      static_for<MB>([&](auto ic) {
        constexpr int mb = decltype(ic)::value;
        f8_lds_wait<2 * (MB - 1 - mb)>(tlo[mb], thi[mb]);
        const u32x4 lo = tlo[mb], hi = thi[mb];
        const i32x8 wf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          const i32x8 hb = {hb_cur[t][0], hb_cur[t][1], hb_cur[t][2], hb_cur[t][3],
                            hb_cur[t][4], hb_cur[t][5], hb_cur[t][6], hb_cur[t][7]};
          oacc[t][mb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, hb, oacc[t][mb], 0, 0, 0, kF8ScaleOne, 0, kF8ScaleOne);
        }
      });

      // ---- epilogue in accumulator order: register jq * 4 + e of row block mb is feature mb * 32 + jq * 8 + hh * 4 + e of
      // token l32. out = bf16(acc * dq2 + b_down + residual), 8-byte pieces.
      const bool want_next = p.amax_next != nullptr;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const int64_t tok = tok0 + t * 32 + l32;
        const bool live = tok < count;
        const int64_t row = f8_token_row(p, count, tok);
        const bf16_t* res_row = p.residual != nullptr ? p.residual + row * p.ldr + hh * 4 : nullptr;
        bf16_t* out_row = p.out + row * p.ldo + hh * 4;
        float ss = 0.f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          bf16x4 rv[4];
          if (res_row != nullptr) {
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) rv[jq] = *reinterpret_cast<const bf16x4*>(res_row + mb * 32 + jq * 8);
          }
#pragma unroll
          for (int jq = 0; jq < 4; ++jq) {
            const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bdown_lds + mb * 32 + jq * 8 + hh * 4);
            bf16x4 ov;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float v = fmaf(oacc[t][mb][jq * 4 + e], dq2, static_cast<float>(bv[e]));
              if (res_row != nullptr) v += static_cast<float>(rv[jq][e]);
              ov[e] = static_cast<bf16_t>(v);
            }
            if (want_next) {  // the rounded output, kept for the statistic below
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float r = static_cast<float>(ov[e]);
                oacc[t][mb][jq * 4 + e] = r;
                ss = fmaf(r, r, ss);
              }
            }
            if (live) *reinterpret_cast<bf16x4*>(out_row + mb * 32 + jq * 8) = ov;
          }
        }
        if (want_next) {
          // amax of what the next layer will quantise: bf16(rmsnorm(out) * w) with its norm weight, or |out| itself. The
          // maximum of the magnitudes is taken on the bf16 bit patterns, two per instruction.
          const float scale = p.next_norm_w != nullptr ? rsqrtf(f8_pair_sum(ss) * (1.0f / D) + p.next_eps) : 1.0f;
          typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
          u16x2 tmax = {0, 0};
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
              bf16x4 wv;
              if (p.next_norm_w != nullptr) wv = *reinterpret_cast<const bf16x4*>(nextw_lds + mb * 32 + jq * 8 + hh * 4);
              bf16x4 nv;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                float v = oacc[t][mb][jq * 4 + e];
                if (p.next_norm_w != nullptr) v = v * scale * static_cast<float>(wv[e]);
                nv[e] = static_cast<bf16_t>(v);
              }
              const u32x2 bits = __builtin_bit_cast(u32x2, nv);
              tmax = __builtin_elementwise_max(tmax, __builtin_bit_cast(u16x2, bits[0] & 0x7fff7fffu));
              tmax = __builtin_elementwise_max(tmax, __builtin_bit_cast(u16x2, bits[1] & 0x7fff7fffu));
            }
          const uint16_t top = tmax[0] > tmax[1] ? tmax[0] : tmax[1];
          const float tm = __builtin_bit_cast(float, static_cast<uint32_t>(top) << 16);
          if (live) nmax = fmaxf(nmax, tm);
        }
      }
    }
    if (p.amax_next != nullptr) f8_block_atomic_max(nmax, p.amax_next, red, wave, lane, NW);
  }
}

__global__ void f8_clear_kernel(float* a, float* b) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    if (a != nullptr) *a = 0.f;
    if (b != nullptr) *b = 0.f;
  }
}

bool f8_ptr_ok(const void* p, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(p) & mask) == 0; }

template <typename K>
int f8_launch(K kernel, const FfnFp8Params& p, int waves, int tokens_per_wg, size_t lds_bytes, hipStream_t s,
              const char* name) {
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);
  const int64_t grid = (p.M + tokens_per_wg - 1) / tokens_per_wg;
  if (grid > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(waves * kWave), lds_bytes, s, p);
  return check_launch(name);
}

}  // namespace
}  // namespace taac

namespace taac {
namespace {

// ---- FP8 preparation of a whole backbone: scales and quantised / packed weights of all blocks in three launches -------
constexpr int kPrepBatch = 16;
struct PrepBatch {
  const bf16_t* w[kPrepBatch][4];   // qkv, out, up, down
  uint8_t* qkv_q[kPrepBatch];
  uint8_t* out_q[kPrepBatch];
  u32x4* ffn_blob[kPrepBatch];
  float* scales[kPrepBatch];        // 4 floats: amax of qkv, out, up, down
};

__global__ __launch_bounds__(256) void f8_fill_zero_kernel(float* a, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) a[i] = 0.f;
}

// blockIdx.y = block * 4 + tensor; grid-stride absolute maximum, one atomic per workgroup.
__global__ __launch_bounds__(256) void f8_weights_amax_kernel(const PrepBatch batch, int D, int F) {
  __shared__ float part[4];
  const int blk = blockIdx.y / 4, which = blockIdx.y % 4;
  const int64_t n = which == 0 ? static_cast<int64_t>(3) * D * D : (which == 1 ? static_cast<int64_t>(D) * D
                                                                                : (which == 2 ? static_cast<int64_t>(2) * F * D
                                                                                              : static_cast<int64_t>(D) * F));
  const bf16x8* w = reinterpret_cast<const bf16x8*>(batch.w[blk][which]);
  float m = 0.f;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n / 8;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const bf16x8 v = w[i];
#pragma unroll
    for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(static_cast<float>(v[e])));
  }
  m = group_max<kWave>(m);
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    atomicMax(reinterpret_cast<unsigned int*>(batch.scales[blk] + which), __float_as_uint(m));
  }
}

// blockIdx.y = block; blockIdx.x walks 16-byte output pieces: the row-major e4m3 copies of qkv and out, then the FFN blob.
__global__ __launch_bounds__(256) void f8_weights_quant_kernel(const PrepBatch batch, int D, int F) {
  const int blk = blockIdx.y;
  const int64_t n_qkv = static_cast<int64_t>(3) * D * D / 16, n_out = static_cast<int64_t>(D) * D / 16;
  int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const float* scales = batch.scales[blk];
  if (gid < n_qkv + n_out) {
    const bool is_out = gid >= n_qkv;
    const int64_t piece = is_out ? gid - n_qkv : gid;
    const bf16_t* src = batch.w[blk][is_out ? 1 : 0] + piece * 16;
    const float scale = fmaxf(scales[is_out ? 1 : 0], 1e-12f) / 448.0f;
    bf16_t v[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = src[e];
    const u32x4 q = {f8_quant4(v, scale), f8_quant4(v + 4, scale), f8_quant4(v + 8, scale), f8_quant4(v + 12, scale)};
    reinterpret_cast<u32x4*>(is_out ? batch.out_q[blk] : batch.qkv_q[blk])[piece] = q;
    return;
  }
  gid -= n_qkv + n_out;
  ffn_fp8_pack_piece(batch.w[blk][2], batch.w[blk][3], scales + 2, scales + 3, batch.ffn_blob[blk], D, F, 1, gid);
}

// max over the listed rows of | bf16(rmsnorm(x, w)) |: 32 lanes per row of 256 features (the scale of a block's first
// dense layer when no producing kernel could deliver it: the embeddings come from outside).
__global__ __launch_bounds__(256) void f8_norm_amax_kernel(const bf16_t* __restrict__ x, int64_t ldx,
                                                           const bf16_t* __restrict__ w, float eps, int64_t M,
                                                           const int32_t* __restrict__ rows,
                                                           const int32_t* __restrict__ n_rows, float* __restrict__ out) {
  __shared__ float part[4];
  const int64_t count = rows != nullptr ? (static_cast<int64_t>(*n_rows) < M ? static_cast<int64_t>(*n_rows) : M) : M;
  const int lane = threadIdx.x % 32;
  float wf[8];
  {
    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(w + lane * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) wf[e] = static_cast<float>(wv[e]);
  }
  float m = 0.f;
  for (int64_t tok = static_cast<int64_t>(blockIdx.x) * 8 + threadIdx.x / 32; tok < count;
       tok += static_cast<int64_t>(gridDim.x) * 8) {
    const int64_t row = rows != nullptr ? static_cast<int64_t>(rows[tok]) : tok;
    const bf16x8 v = *reinterpret_cast<const bf16x8*>(x + row * ldx + lane * 8);
    float f[8], ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      f[e] = static_cast<float>(v[e]);
      ss = fmaf(f[e], f[e], ss);
    }
    const float scale = rsqrtf(group_sum<32>(ss) * (1.0f / 256.0f) + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(static_cast<float>(static_cast<bf16_t>(f[e] * scale * wf[e]))));
  }
  m = group_max<kWave>(m);
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    if (m > __builtin_nontemporal_load(out)) atomicMax(reinterpret_cast<unsigned int*>(out), __float_as_uint(m));
  }
}

}  // namespace

// Scales (4 floats per block: qkv, out, up, down; zeroed by the caller) and the e4m3 weights of n backbone blocks: row-major qkv / out copies and
// the feed-forward blob (gate first). D = 256, F a multiple of 64.
int prepare_backbone_fp8(const taac_block_weights* blocks, int n, int32_t D, int32_t F, float* const* scales,
                         void* const* qkv_q, void* const* out_q, void* const* ffn_blob, hipStream_t s, const char* name) {
  for (int base = 0; base < n; base += kPrepBatch) {
    PrepBatch batch{};
    const int m = n - base < kPrepBatch ? n - base : kPrepBatch;
    for (int i = 0; i < m; ++i) {
      const taac_block_weights& w = blocks[base + i];
      const void* ptrs[4] = {w.qkv_weight, w.out_weight, w.up_weight, w.down_weight};
      for (int t = 0; t < 4; ++t) {
        if (!ptrs[t] || (reinterpret_cast<uintptr_t>(ptrs[t]) & 15u))
          return set_error(TAAC_ERR_UNSUPPORTED, "%s: weights must be given and 16-byte aligned", name);
        batch.w[i][t] = static_cast<const bf16_t*>(ptrs[t]);
      }
      batch.qkv_q[i] = static_cast<uint8_t*>(qkv_q[base + i]);
      batch.out_q[i] = static_cast<uint8_t*>(out_q[base + i]);
      batch.ffn_blob[i] = static_cast<u32x4*>(ffn_blob[base + i]);
      batch.scales[i] = scales[base + i];
    }
    hipLaunchKernelGGL(f8_weights_amax_kernel, dim3(16, 4 * m), dim3(256), 0, s, batch, D, F);
    const int64_t pieces = (static_cast<int64_t>(4) * D * D + taac_ffn_fp8_packed_bytes(D, F)) / 16;
    hipLaunchKernelGGL(f8_weights_quant_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256), m), dim3(256), 0, s, batch,
                       D, F);
    const int rc = check_launch(name);
    if (rc != TAAC_OK) return rc;
  }
  return TAAC_OK;
}

// *out (zeroed by the caller) = max over the (listed) rows of | bf16(rmsnorm(x, w, eps)) |, rows of 256 bf16 features.
int fill_zero(float* p, int n, hipStream_t s, const char* name) {
  hipLaunchKernelGGL(f8_fill_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, s, p, n);
  return check_launch(name);
}

int rmsnorm_amax_256(const void* x, int64_t ldx, const void* w, float eps, int64_t M, const int32_t* rows,
                     const int32_t* n_rows, float* out, hipStream_t s, const char* name) {
  if (M > 0) {
    int64_t grid = (M + 7) / 8;
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(f8_norm_amax_kernel, dim3(static_cast<uint32_t>(grid)), dim3(256), 0, s, static_cast<const bf16_t*>(x),
                       ldx, static_cast<const bf16_t*>(w), eps, M, rows, n_rows, out);
  }
  return check_launch(name);
}

}  // namespace taac

extern "C" int64_t taac_ffn_fp8_packed_bytes(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % taac::kF8Chunk != 0) return -1;
  return static_cast<int64_t>(3) * D * F + static_cast<int64_t>(64) * D;  // the stream of steps + the tail fragments
}

extern "C" int taac_ffn_fp8_pack_weights(const void* w_up, const void* w_down, const float* amax_up,
                                         const float* amax_down, void* packed, int32_t D, int32_t F, int gate_first,
                                         void* stream) {
  using namespace taac;
  const char* name = "taac_ffn_fp8_pack_weights";
  if (taac_ffn_fp8_packed_bytes(D, F) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D must be 128 or 256 and F a positive multiple of 64", name);
  if (!w_up || !w_down || !amax_up || !amax_down || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!f8_ptr_ok(packed, 15)) return set_error(TAAC_ERR_UNSUPPORTED, "%s: the blob must be 16-byte aligned", name);
  const int64_t pieces = taac_ffn_fp8_packed_bytes(D, F) / 16;
  hipLaunchKernelGGL(ffn_fp8_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const bf16_t*>(w_up), static_cast<const bf16_t*>(w_down), amax_up, amax_down,
                     static_cast<u32x4*>(packed), D, F, gate_first ? 1 : 0);
  return check_launch(name);
}

extern "C" int taac_swiglu_ffn_fp8_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps,
                                       const void* packed_weights, const void* b_up, const void* b_down,
                                       const float* amax_x, const float* amax_up, const float* amax_down,
                                       float* amax_hidden, const void* residual, int64_t ldr, void* out, int64_t ldo,
                                       int64_t M, int32_t D, int32_t F, int gate_first, const int32_t* rows,
                                       const int32_t* n_rows, const void* next_norm_weight, float next_eps,
                                       float* amax_next, void* stream) {
  using namespace taac;
  const char* name = "taac_swiglu_ffn_fp8_fwd";
  if (M < 0 || D <= 0 || F <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, D and F > 0", name);
  if (taac_ffn_fp8_packed_bytes(D, F) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D must be 128 or 256 and F a multiple of 64 (got D=%d, F=%d)", name, D, F);
  if (ldx < D || ldo < D || (residual && ldr < D) || ldx % 8 || ldo % 8 || (residual && ldr % 8))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (!amax_x || !amax_up || !amax_down || !amax_hidden)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the four scale pointers are required", name);
  if ((rows == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows and n_rows must be given together", name);
  if (next_norm_weight && !amax_next)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: next_norm_weight without amax_next", name);
  hipStream_t s = as_stream(stream);
  if (M == 0) {
    hipLaunchKernelGGL(f8_clear_kernel, dim3(1), dim3(kWave), 0, s, amax_hidden, amax_next);
    return check_launch(name);
  }
  if (!x || !out || !packed_weights) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (rows && M > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: a row index covers at most 2^31 rows", name);
  if (!f8_ptr_ok(x, 15) || !f8_ptr_ok(out, 7) || !f8_ptr_ok(residual, 7) || !f8_ptr_ok(norm_weight, 15) ||
      !f8_ptr_ok(b_up, 1) || !f8_ptr_ok(b_down, 15) || !f8_ptr_ok(packed_weights, 15) || !f8_ptr_ok(next_norm_weight, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int KS = D / 64, MB = D / 32;
  const size_t tail = static_cast<size_t>(3 * D) * 2 + 128 + (b_up != nullptr ? static_cast<size_t>(2 * F) * 4 : 0);
  const size_t lds1 = static_cast<size_t>(2 * 2 * KS) * kF8Frag + tail;              // two buffers of two sub-chunks, up only
  const size_t lds2 = static_cast<size_t>(2 * 2 * (KS + MB / 4)) * kF8Frag + tail;   // ... with their down fragments
  if (lds2 > 80 * 1024)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: F=%d does not leave room for two workgroups per compute unit", name, F);
  FfnFp8Params p{};
  p.x = static_cast<const bf16_t*>(x);
  p.norm_w = static_cast<const bf16_t*>(norm_weight);
  p.packed = static_cast<const uint8_t*>(packed_weights);
  p.b_up = static_cast<const bf16_t*>(b_up);
  p.b_down = static_cast<const bf16_t*>(b_down);
  p.residual = static_cast<const bf16_t*>(residual);
  p.out = static_cast<bf16_t*>(out);
  p.next_norm_w = static_cast<const bf16_t*>(next_norm_weight);
  p.amax_x = amax_x;
  p.amax_up = amax_up;
  p.amax_down = amax_down;
  p.amax_hidden = amax_hidden;
  p.amax_next = amax_next;
  p.M = M;
  p.ldx = ldx;
  p.ldr = ldr;
  p.ldo = ldo;
  p.F = F;
  p.gate_first = gate_first ? 1 : 0;
  p.eps = eps;
  p.next_eps = next_eps;
  p.rows = rows;
  p.n_rows = n_rows;
  int rc = TAAC_OK;
  if (!maxima_precleared) {
    hipLaunchKernelGGL(f8_clear_kernel, dim3(1), dim3(kWave), 0, s, amax_hidden, amax_next);
    if ((rc = check_launch(name)) != TAAC_OK) return rc;
  }
// pass 1: 4 wavefronts x 2 tiles; pass 2: 4 wavefronts x 1 tile; two workgroups per compute unit
#define TAAC_F8_FFN(DD, BB)                                                                                             \
  do {                                                                                                                  \
    if ((rc = f8_launch(swiglu_ffn_fp8_kernel<DD, 2, 4, false, BB>, p, 4, 4 * 64, lds1, s, name)) != TAAC_OK) return rc; \
    return f8_launch(swiglu_ffn_fp8_kernel<DD, 1, 4, true, BB>, p, 4, 4 * 32, lds2, s, name);                           \
  } while (0)
  if (D == 256) {
    if (b_up != nullptr) TAAC_F8_FFN(256, true);
    TAAC_F8_FFN(256, false);
  }
  if (b_up != nullptr) TAAC_F8_FFN(128, true);
  TAAC_F8_FFN(128, false);
#undef TAAC_F8_FFN
}
