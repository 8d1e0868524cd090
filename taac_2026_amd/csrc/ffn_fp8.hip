// Token-stationary fused SwiGLU feed-forward with FP8 (OCP e4m3fn, per-tensor scales) MFMA operands for gfx950:
//   h   = norm_weight ? bf16(rmsnorm(x, norm_weight)) : x                      quantised with scale amax_x / 448
//   g,u = chunk2( (q(h) q(w_up)^T) * s_x * s_up + b_up )                       fp32
//   hid = bf16( silu(g) * u )                                                  quantised with scale amax_hidden / 448
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
// Scheme (as the bf16 kernel of ffn.hip): a wavefront owns 32 tokens (pass 1: 64) for the whole kernel and keeps their
// quantised rows as MFMA B operands of v_mfma_scale_f32_32x32x64_f8f6f4 (lane (l32, hh) holds the 32 bytes
// k = 64 ks + 32 hh .. + 31 of token l32); the weights stream L2 -> LDS by DMA in fragment order (2 KB fragments =
// 32 rows x 64 k, written as two 1 KB halves) through a ring of buffers, one barrier per 64 hidden units.
// A chunk of 64 hidden units is four sub-chunks of 16: the up fragment of a sub-chunk stacks 16 gated rows on their 16
// partner rows, so one accumulator holds g (registers 0..7) and u (8..15) of eight hidden units of the lane's token;
// silu(g) * u of the four sub-chunks are the lane's 32 bytes of the down projection's B operand (the k order of the
// packed W_down fragments follows that register order). The down projection of a chunk is issued one chunk late,
// two MFMAs behind every sub-chunk of the next one, with that sub-chunk's activation arithmetic between them.
#include <cstdlib>

#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kF8Frag = 2048;     // bytes of one 32 x 64 e4m3 fragment
constexpr int kF8Waves = 8;
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

__device__ __forceinline__ float f8_silu(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
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
// Blob: chunk c (hidden units 64 c .. 64 c + 63) = 4 * D / 64 up fragments (sub-chunk s, k-step ks) at index
// s * (D / 64) + ks, then D / 32 down fragments (row block mb). A fragment is the LDS image: half h (1 KB) holds for
// lane l the 16 bytes k = 32 * (l / 32) + 16 h .. + 15 of row l % 32.
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

__global__ __launch_bounds__(256) void ffn_fp8_pack_kernel(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                                           const float* __restrict__ amax_up,
                                                           const float* __restrict__ amax_down, u32x4* __restrict__ packed,
                                                           int D, int F, int gate_first) {
  const int KS = D / 64, MB = D / 32, UPF = 4 * KS, CFRAG = UPF + MB;
  const int64_t total = static_cast<int64_t>(3) * D * F / 16;  // 16-byte pieces
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int lane = static_cast<int>(gid % 64);
  const int half = static_cast<int>((gid / 64) % 2);
  const int f = static_cast<int>((gid / 128) % CFRAG);
  const int64_t chunk = gid / 128 / CFRAG;
  const int l32 = lane % 32, hh = lane / 32;
  bf16_t v[16];
  float scale;
  if (f < UPF) {
    const int s = f / KS, ks = f % KS;
    const int64_t row = ((l32 < 16) == (gate_first != 0) ? 0 : F) + chunk * kF8Chunk + 16 * s + f8_unit_of_slot(l32 & 15);
    const bf16_t* src = w_up + row * D + ks * 64 + hh * 32 + half * 16;
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = src[e];
    scale = fmaxf(*amax_up, 1e-12f) / 448.0f;
  } else {
    const int mb = f - UPF;
    const bf16_t* src = w_down + static_cast<int64_t>(mb * 32 + l32) * F + chunk * kF8Chunk;
#pragma unroll
    for (int b = 0; b < 16; ++b) v[b] = src[16 * (2 * half + b / 8) + 8 * hh + b % 8];
    scale = fmaxf(*amax_down, 1e-12f) / 448.0f;
  }
  const u32x4 q = {f8_quant4(v, scale), f8_quant4(v + 4, scale), f8_quant4(v + 8, scale), f8_quant4(v + 12, scale)};
  packed[gid] = q;
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

// Up-projection bias in accumulator order: entry (chunk * 4 + s) * 16 + 8 * half + 8-run: for sub-chunk s of a chunk,
// dst[(chunk * 4 + s) * 32 + hh * 16 + j] = bias of the gated unit 8 hh + j (j < 8), + 8: of its partner.
__device__ __forceinline__ void f8_stage_up_bias(const bf16_t* b_up, bf16_t* dst, int F, int gate_first, int tid, int nthreads) {
  for (int i = tid; i < 2 * F; i += nthreads) {
    const int sub = i / 32, r = i % 32, hh = r / 16, j = r % 16;
    const int unit = sub * 16 + 8 * hh + (j % 8);
    const int src = ((j < 8) == (gate_first != 0) ? 0 : F) + unit;
    dst[i] = b_up != nullptr ? b_up[src] : static_cast<bf16_t>(0.f);
  }
}

// ---- the kernel -------------------------------------------------------------------------------------------------------
// PASS2 = false: TT tiles of 32 tokens per wavefront, up projection + activation, max |hid| -> amax_hidden.
// PASS2 = true:  one tile per wavefront, the whole layer.
// LDS: [NBUF weight buffers][b_up in accumulator order (2F) | b_down (D) | norm weight (D) | next norm weight (D)][8 floats]
template <int D, int TT, bool PASS2>
__global__ __launch_bounds__(kF8Waves* kWave, 1) void swiglu_ffn_fp8_kernel(const FfnFp8Params p) {
  static_assert(!PASS2 || TT == 1, "the full layer keeps one tile's output accumulator in registers");
  constexpr int KS = D / 64;                    // k-steps of the up projection
  constexpr int MB = D / 32;                    // row blocks of the down projection
  constexpr int UPF = 4 * KS;                   // up fragments per chunk
  constexpr int BLOB_FRAG = UPF + MB;           // fragments per chunk in the blob
  constexpr int CFRAG = PASS2 ? BLOB_FRAG : UPF;  // fragments staged per chunk
  constexpr int kBuf = CFRAG * kF8Frag;
  constexpr int NBUF = PASS2 ? 3 : 2;
  constexpr int DPW = CFRAG * 2 / kF8Waves;     // 1 KB DMA instructions per wavefront and chunk
  static_assert(CFRAG * 2 % kF8Waves == 0, "the transfers of a chunk divide over the wavefronts");
  constexpr int DPS = MB / 4;                   // down MFMAs behind every sub-chunk
  constexpr int SFRAG = KS + (PASS2 ? DPS : 0);  // fragments consumed per sub-chunk
  constexpr int NSTREAM = 4 * SFRAG;            // fragments consumed per chunk
  constexpr int P = 4;                          // fragments in flight
  constexpr int kTokPerWg = kF8Waves * 32 * TT;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(smem + NBUF * kBuf);
  const int F = p.F;
  bf16_t* bdown_lds = bias_lds + 2 * F;
  bf16_t* normw_lds = bdown_lds + D;
  bf16_t* nextw_lds = normw_lds + D;
  float* red = reinterpret_cast<float*>(nextw_lds + D);

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
  const int nchunks = F / kF8Chunk;

  auto stage = [&](int chunk, int buf) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
    const uint8_t* src = p.packed + (static_cast<int64_t>(chunk) * BLOB_FRAG * 2 + wave * DPW) * 1024;
    uint8_t* dst = smem + buf * kBuf + wave * (DPW * 1024);
#pragma unroll
    for (int i = 0; i < DPW; ++i) lds_dma16_offset(src + i * 1024, lane_off, dst + i * 1024);
  };

  stage(0, 0);
  f8_stage_up_bias(p.b_up, bias_lds, F, p.gate_first, tid, kF8Waves * kWave);
  stage_bias(p.b_down, bdown_lds, D, tid, kF8Waves * kWave);
  stage_bias(p.norm_w, normw_lds, D, tid, kF8Waves * kWave);
  stage_bias(p.next_norm_w, nextw_lds, D, tid, kF8Waves * kWave);

  const float amax_x = fmaxf(*p.amax_x, 1e-12f);
  const float amax_up = fmaxf(*p.amax_up, 1e-12f);
  const float dq1 = (amax_x / 448.0f) * (amax_up / 448.0f);
  float inv_scale_h = 0.f, dq2 = 0.f;
  if (PASS2) {
    const float amax_h = fmaxf(*p.amax_hidden, 1e-12f);
    inv_scale_h = 448.0f / amax_h;
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

  f32x16 oacc[PASS2 ? MB : 1];
  if (PASS2) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) oacc[mb][j] = 0.f;
  }
  const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float hmax = 0.f;
  // hb_cur: the quantised hidden state of the previous chunk (B operand of its pending down projection); hb_nxt: the
  // one being assembled. Before the first chunk hb_cur is zero and multiplies chunk 0's own (finite) down fragments.
  int hb_cur[8], hb_nxt[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) hb_cur[i] = hb_nxt[i] = 0;
  // pass 1 pipelines the activation of a sub-chunk behind the products of the next one: two accumulator sets
  f32x16 gu[PASS2 ? 1 : 2][TT];
#pragma unroll
  for (int a = 0; a < (PASS2 ? 1 : 2); ++a)
#pragma unroll
    for (int t = 0; t < TT; ++t) gu[a][t] = zero16;

  const uint32_t smem_off = lds_offset(smem) + lane * 16;
  const bf16_t* bias_lane = bias_lds + hh * 16;

  // silu(g) * u of the eight hidden units a lane holds of one sub-chunk (registers j and 8 + j), rounded to bf16.
  auto activate = [&](const f32x16& acc, const bf16x8& bg, const bf16x8& bu, int j) -> float {
    const float g = fmaf(acc[j], dq1, static_cast<float>(bg[j]));
    const float u = fmaf(acc[8 + j], dq1, static_cast<float>(bu[j]));
    return static_cast<float>(static_cast<bf16_t>(f8_silu(g) * u));
  };

  int buf = 0;
  uint32_t wb_prev = smem_off;
  for (int c = 0; c < nchunks; ++c) {
    if (c + 1 < nchunks) stage(c + 1, buf == NBUF - 1 ? 0 : buf + 1);
    const uint32_t wb = smem_off + buf * kBuf;
    if (active) {
      u32x4 rlo[P], rhi[P];
      // fragment i of the chunk's stream: sub-chunk s = i / SFRAG; r < KS: up fragment (s, r); else down fragment
      // s * DPS + r - KS of the previous chunk (in the previous buffer)
      auto read_stream = [&](auto ic, int slot) {
        constexpr int i = decltype(ic)::value;
        constexpr int s = i / SFRAG, r = i % SFRAG;
        if constexpr (r < KS) {
          f8_lds_read16<(s * KS + r) * kF8Frag>(rlo[slot], wb);
          f8_lds_read16<(s * KS + r) * kF8Frag + 1024>(rhi[slot], wb);
        } else {
          f8_lds_read16<(UPF + s * DPS + r - KS) * kF8Frag>(rlo[slot], wb_prev);
          f8_lds_read16<(UPF + s * DPS + r - KS) * kF8Frag + 1024>(rhi[slot], wb_prev);
        }
      };
      static_for<P>([&](auto ic) { read_stream(ic, decltype(ic)::value); });
      const bf16_t* bias_chunk = bias_lane + c * (4 * 32);
      static_for<NSTREAM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        constexpr int s = i / SFRAG, r = i % SFRAG;
        constexpr int after = 2 * (P - 1 < NSTREAM - 1 - i ? P - 1 : NSTREAM - 1 - i);
        f8_lds_wait<after>(rlo[i % P], rhi[i % P]);
        const u32x4 lo = rlo[i % P], hi = rhi[i % P];
        const i32x8 wf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        if constexpr (r < KS) {
          // ---- up projection of sub-chunk s ----------------------------------------------------------------------------
          constexpr int a = PASS2 ? 0 : s % 2;
#pragma unroll
          for (int t = 0; t < TT; ++t) {
            gu[a][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, xq[t][r], r == 0 ? zero16 : gu[a][t], 0, 0, 0,
                                                                         kF8ScaleOne, 0, kF8ScaleOne);
            asm volatile("" : "+v"(gu[a][t]));
          }
        } else {
          // ---- down projection of the previous chunk, row block s * DPS + r - KS ----------------------------------------
          constexpr int mb = s * DPS + r - KS;
          const i32x8 hb = {hb_cur[0], hb_cur[1], hb_cur[2], hb_cur[3], hb_cur[4], hb_cur[5], hb_cur[6], hb_cur[7]};
          oacc[PASS2 ? mb : 0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, hb, oacc[PASS2 ? mb : 0], 0, 0, 0,
                                                                                  kF8ScaleOne, 0, kF8ScaleOne);
          asm volatile("" : "+v"(oacc[PASS2 ? mb : 0]));
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i + P < NSTREAM) read_stream(std::integral_constant<int, i + P>{}, i % P);
        if constexpr (PASS2 && r >= KS) {
          // ---- activation of sub-chunk s (its products were issued before the down MFMAs of this group): the 8 values
          // of a lane are spread over the DPS down MFMAs; values 4k .. 4k+3 make dword 2 s + k of the B operand ----------
          constexpr int d = r - KS;
          const bf16x8 bg = *reinterpret_cast<const bf16x8*>(bias_chunk + s * 32);
          const bf16x8 bu = *reinterpret_cast<const bf16x8*>(bias_chunk + s * 32 + 8);
#pragma unroll
          for (int k = d * 2 / DPS; k < (d + 1) * 2 / DPS; ++k) {
            float h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = activate(gu[0][0], bg, bu, 4 * k + e) * inv_scale_h;
            int w = f8_pack2<false>(h[0], h[1], 0);
            hb_nxt[2 * s + k] = f8_pack2<true>(h[2], h[3], w);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (!PASS2 && r == KS - 1) {
          // ---- pass 1: activation of the PREVIOUS sub-chunk (its accumulator set is the other one; before the very first
          // sub-chunk that set is zero and the bias slot read is that of sub-chunk 3 of the previous chunk) ----------------
          constexpr int prev = (s + 3) % 4, a = (s + 1) % 2;
          const bf16_t* bsrc = s == 0 ? bias_chunk - 4 * 32 + prev * 32 : bias_chunk + prev * 32;
          if (s != 0 || c > 0) {
            const bf16x8 bg = *reinterpret_cast<const bf16x8*>(bsrc);
            const bf16x8 bu = *reinterpret_cast<const bf16x8*>(bsrc + 8);
#pragma unroll
            for (int t = 0; t < TT; ++t)
#pragma unroll
              for (int j = 0; j < 8; ++j) hmax = fmaxf(hmax, fabsf(activate(gu[a][t], bg, bu, j)));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      if (PASS2) {
#pragma unroll
        for (int i = 0; i < 8; ++i) hb_cur[i] = hb_nxt[i];
      }
    }
    vm_wait<0>();  // the next chunk's weights (the only vector-memory operations of the loop)
    __syncthreads();
    wb_prev = wb;
    buf = buf == NBUF - 1 ? 0 : buf + 1;
  }

  if constexpr (!PASS2) {
    if (active) {  // the last sub-chunk's activation is still pending (accumulator set 1)
      const bf16_t* bsrc = bias_lane + (nchunks - 1) * (4 * 32) + 3 * 32;
      const bf16x8 bg = *reinterpret_cast<const bf16x8*>(bsrc);
      const bf16x8 bu = *reinterpret_cast<const bf16x8*>(bsrc + 8);
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) hmax = fmaxf(hmax, fabsf(activate(gu[1][t], bg, bu, j)));
    }
    f8_block_atomic_max(active ? hmax : 0.f, p.amax_hidden, red, wave, lane, kF8Waves);
    return;
  } else {
    // ---- the down projection of the last chunk is still pending; its fragments are in the last chunk's buffer ------------
    float nmax = 0.f;
    if (active) {
      u32x4 tlo[MB], thi[MB];
      static_for<MB>([&](auto ic) {
        constexpr int mb = decltype(ic)::value;
        f8_lds_read16<(UPF + mb) * kF8Frag>(tlo[mb], wb_prev);
        f8_lds_read16<(UPF + mb) * kF8Frag + 1024>(thi[mb], wb_prev);
      });
      const i32x8 hb = {hb_cur[0], hb_cur[1], hb_cur[2], hb_cur[3], hb_cur[4], hb_cur[5], hb_cur[6], hb_cur[7]};
      static_for<MB>([&](auto ic) {
        constexpr int mb = decltype(ic)::value;
        f8_lds_wait<2 * (MB - 1 - mb)>(tlo[mb], thi[mb]);
        const u32x4 lo = tlo[mb], hi = thi[mb];
        const i32x8 wf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        oacc[mb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, hb, oacc[mb], 0, 0, 0, kF8ScaleOne, 0, kF8ScaleOne);
      });

      // ---- epilogue in accumulator order: register jq * 4 + e of row block mb is feature mb * 32 + jq * 8 + hh * 4 + e of
      // token l32. out = bf16(acc * dq2 + b_down + residual), 8-byte pieces.
      const int64_t tok = tok0 + l32;
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
            float v = fmaf(oacc[mb][jq * 4 + e], dq2, static_cast<float>(bv[e]));
            if (res_row != nullptr) v += static_cast<float>(rv[jq][e]);
            ov[e] = static_cast<bf16_t>(v);
            const float r = static_cast<float>(ov[e]);
            oacc[mb][jq * 4 + e] = r;  // the rounded output, kept for the statistic below
            ss = fmaf(r, r, ss);
          }
          if (live) *reinterpret_cast<bf16x4*>(out_row + mb * 32 + jq * 8) = ov;
        }
      }
      if (p.amax_next != nullptr) {
        // amax of what the next layer will quantise: bf16(rmsnorm(out) * w) with its norm weight, or |out| itself
        const float scale = p.next_norm_w != nullptr ? rsqrtf(f8_pair_sum(ss) * (1.0f / D) + p.next_eps) : 1.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int jq = 0; jq < 4; ++jq) {
            bf16x4 wv;
            if (p.next_norm_w != nullptr) wv = *reinterpret_cast<const bf16x4*>(nextw_lds + mb * 32 + jq * 8 + hh * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float v = oacc[mb][jq * 4 + e];
              if (p.next_norm_w != nullptr) v = static_cast<float>(static_cast<bf16_t>(v * scale * static_cast<float>(wv[e])));
              nmax = fmaxf(nmax, fabsf(v));
            }
          }
        if (!live) nmax = 0.f;
      }
    }
    if (p.amax_next != nullptr) f8_block_atomic_max(nmax, p.amax_next, red, wave, lane, kF8Waves);
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
int f8_launch(K kernel, const FfnFp8Params& p, int tokens_per_wg, size_t lds_bytes, hipStream_t s, const char* name) {
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);
  const int64_t grid = (p.M + tokens_per_wg - 1) / tokens_per_wg;
  if (grid > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(kF8Waves * kWave), lds_bytes, s, p);
  return check_launch(name);
}

}  // namespace
}  // namespace taac

extern "C" int64_t taac_ffn_fp8_packed_bytes(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % taac::kF8Chunk != 0) return -1;
  return static_cast<int64_t>(3) * D * F;
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
  const int64_t pieces = static_cast<int64_t>(3) * D * F / 16;
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
  const size_t tail = static_cast<size_t>(2 * F + 3 * D) * 2 + 64;
  const size_t lds1 = static_cast<size_t>(2 * 4 * KS) * kF8Frag + tail;
  const size_t lds2 = static_cast<size_t>(3 * (4 * KS + MB)) * kF8Frag + tail;
  if (lds2 > 160 * 1024) return set_error(TAAC_ERR_UNSUPPORTED, "%s: F=%d does not fit the LDS", name, F);
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
  hipLaunchKernelGGL(f8_clear_kernel, dim3(1), dim3(kWave), 0, s, amax_hidden, amax_next);
  int rc = check_launch(name);
  if (rc != TAAC_OK) return rc;
  if (D == 256) {
    if ((rc = f8_launch(swiglu_ffn_fp8_kernel<256, 2, false>, p, kF8Waves * 64, lds1, s, name)) != TAAC_OK) return rc;
    return f8_launch(swiglu_ffn_fp8_kernel<256, 1, true>, p, kF8Waves * 32, lds2, s, name);
  }
  if ((rc = f8_launch(swiglu_ffn_fp8_kernel<128, 2, false>, p, kF8Waves * 64, lds1, s, name)) != TAAC_OK) return rc;
  return f8_launch(swiglu_ffn_fp8_kernel<128, 1, true>, p, kF8Waves * 32, lds2, s, name);
}
