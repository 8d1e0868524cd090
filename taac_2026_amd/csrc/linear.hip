// Dense layers of the backbone block on gfx950 MFMA: out = epilogue(a @ w^T + bias), bf16 or fp8 operands,
// fp32 accumulation, bf16 output.
//
// Tiling
//   Workgroup tile = 128 tokens x 128 output features, 4 wavefronts in a 2 x 2 arrangement, each owning
//   64 tokens x 64 features as 2 x 2 v_mfma_f32_32x32x16 tiles. The reduction dimension is walked in slabs of 64
//   (bf16) or 128 (fp8) elements staged through LDS; the next slab's global loads are issued before the current
//   slab's MFMAs so that they overlap.
//   The product is formed transposed, C^T[feature, token] = W A^T: the weight rows are the MFMA A operand and the
//   token rows the B operand, both read along their contiguous K axis. In the accumulator layout a lane then owns
//   one token and runs of 4 consecutive output features, so bias / residual / SiLU-gate epilogues and the bf16
//   stores work on 8-byte pieces of a row.
//   Logical workgroup ids walk the feature tiles of one token tile first and are remapped so that neighbours share
//   an accelerator die: the token slab is fetched from HBM once and re-read from that die's L2.
//
// SwiGLU epilogue: a workgroup's 128 weight rows are 64 gate rows [n0, n0+64) and the 64 matching value rows
// [F+n0, F+n0+64); each wavefront holds gate and value of the same (token, feature) in the same lane and
// register index, so silu(g) * u is formed in registers and the [M, 2F] projection is never written.
// Follows SwiGLUFeedForward.forward (experiments/symbiosis/backbone.py:19-21): gate, value = up(x).chunk(2, -1).
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kThreads = 256;
constexpr int kBM = 128;  // tokens per workgroup
constexpr int kBN = 128;  // weight rows per workgroup

struct LinearParams {
  const void* a;
  const void* w;
  const void* bias;      // 16-bit elements of the kernel's output type
  const void* residual;
  void* out;
  const float* amax_a;  // fp8 only
  const float* amax_w;  // fp8 only
  int64_t lda, ldo, M;
  int32_t N, K;
  int32_t F;  // SwiGLU: N / 2
  int32_t gate_first;
  uint32_t ntiles, total;
};

__device__ __forceinline__ float silu_f(float x) {
  // x * sigmoid(x) with the hardware exp2 / rcp
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// Accumulator -> bf16 output for one wavefront. acc[ni][mi][j]: feature sub-tile ni, token sub-tile mi,
// j -> feature (j/4)*8 + hh*4 + j%4 inside the 32-feature sub-tile, token l32 inside the 32-token sub-tile.
template <int EPI, typename T = bf16_t>
__device__ __forceinline__ void store_tile(const LinearParams& p, f32x16 (&acc)[2][2], float dq, int64_t m0, int n0,
                                           int wt, int wn, int l32, int hh) {
  typedef typename Vec8<T>::half_type vec4_t;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int64_t row = m0 + wt * 64 + mi * 32 + l32;
    if (row >= p.M) continue;
    T* orow = reinterpret_cast<T*>(p.out) + row * p.ldo;
    const T* rrow = (EPI == TAAC_EPI_RESIDUAL) ? reinterpret_cast<const T*>(p.residual) + row * p.ldo : nullptr;
    const T* bias = reinterpret_cast<const T*>(p.bias);
    if (EPI == TAAC_EPI_SWIGLU) {
#pragma unroll
      for (int jq = 0; jq < 4; ++jq) {
        const int col = n0 + wn * 32 + jq * 8 + hh * 4;  // output feature, < F
        if (col >= p.F) continue;
        float g[4], u[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          g[e] = acc[0][mi][jq * 4 + e] * dq;
          u[e] = acc[1][mi][jq * 4 + e] * dq;
        }
        if (p.bias != nullptr) {
          const vec4_t bg = *reinterpret_cast<const vec4_t*>(bias + col);
          const vec4_t bu = *reinterpret_cast<const vec4_t*>(bias + p.F + col);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            g[e] += static_cast<float>(bg[e]);
            u[e] += static_cast<float>(bu[e]);
          }
        }
        vec4_t ov;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          ov[e] = static_cast<T>(p.gate_first ? silu_f(g[e]) * u[e] : g[e] * silu_f(u[e]));
        *reinterpret_cast<vec4_t*>(orow + col) = ov;
      }
    } else {
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          const int col = n0 + wn * 64 + ni * 32 + jq * 8 + hh * 4;
          if (col >= p.N) continue;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[ni][mi][jq * 4 + e] * dq;
          if (p.bias != nullptr) {
            const vec4_t bv = *reinterpret_cast<const vec4_t*>(bias + col);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += static_cast<float>(bv[e]);
          }
          if (EPI == TAAC_EPI_RESIDUAL) {
            const vec4_t rv = *reinterpret_cast<const vec4_t*>(rrow + col);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += static_cast<float>(rv[e]);
          }
          vec4_t ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(v[e]);
          *reinterpret_cast<vec4_t*>(orow + col) = ov;
        }
      }
    }
  }
}

// Row of w held by LDS weight-tile row r of the workgroup whose first output feature is n0.
template <int EPI>
__device__ __forceinline__ int weight_row(const LinearParams& p, int n0, int r) {
  if (EPI == TAAC_EPI_SWIGLU) return r < 64 ? n0 + r : p.F + n0 + (r - 64);
  return n0 + r;
}
template <int EPI>
__device__ __forceinline__ bool weight_row_ok(const LinearParams& p, int n0, int r) {
  if (EPI == TAAC_EPI_SWIGLU) return n0 + (r & 63) < p.F;
  return n0 + r < p.N;
}

// ------------------------------------------------------------------------------------------------------------------
// bf16 operands
// ------------------------------------------------------------------------------------------------------------------
template <typename T>
struct Mfma16;
template <>
struct Mfma16<bf16_t> {
  static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16<f16_t> {  // the staged 16-byte pieces are opaque: reinterpret them as eight halves
  static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// T: the 16-bit element type of operands, bias, residual and output (bf16_t or f16_t); the staging below moves opaque
// 16-byte pieces, only the MFMA and the epilogue depend on it.
template <int EPI, typename T = bf16_t>
__global__ __launch_bounds__(kThreads) void linear_bf16_kernel(const LinearParams p) {
  constexpr int BK = 64;
  constexpr int STR = BK + 8;          // LDS row stride in elements (+16 bytes)
  constexpr int CH = BK / 8;           // 128-bit chunks per tile row
  constexpr int LD = kBM * CH / kThreads;  // chunks per thread per operand (4)
  __shared__ __attribute__((aligned(16))) bf16_t sA[kBM * STR];
  __shared__ __attribute__((aligned(16))) bf16_t sW[kBN * STR];

  const uint32_t logical = xcd_remap(blockIdx.x, p.total);
  const int nt = static_cast<int>(logical % p.ntiles);
  const int64_t mt = logical / p.ntiles;
  const int64_t m0 = mt * kBM;
  const int n0 = nt * (EPI == TAAC_EPI_SWIGLU ? 64 : kBN);

  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int wt = wave % 2;  // token half
  const int wn = wave / 2;  // feature half

  const bf16_t* A = static_cast<const bf16_t*>(p.a);
  const bf16_t* W = static_cast<const bf16_t*>(p.w);

  bf16x8 zero_vec;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero_vec[e] = static_cast<bf16_t>(0.f);

  // Per-thread staging slots: chunk c = tid + 256*i -> tile row c / CH, 8-element column c % CH.
  const bf16_t* a_src[LD];
  const bf16_t* w_src[LD];
  int lds_off[LD];
  int col_off[LD];
#pragma unroll
  for (int i = 0; i < LD; ++i) {
    const int cidx = tid + kThreads * i;
    const int r = cidx / CH;
    const int c8 = cidx % CH;
    lds_off[i] = r * STR + c8 * 8;
    col_off[i] = c8 * 8;
    a_src[i] = (m0 + r < p.M) ? A + (m0 + r) * p.lda + c8 * 8 : nullptr;
    w_src[i] = weight_row_ok<EPI>(p, n0, r) ? W + static_cast<int64_t>(weight_row<EPI>(p, n0, r)) * p.K + c8 * 8
                                             : nullptr;
  }

  bf16x8 ra[LD], rw[LD];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < LD; ++i) {
      const bool kin = k0 + col_off[i] < p.K;
      ra[i] = (a_src[i] != nullptr && kin) ? *reinterpret_cast<const bf16x8*>(a_src[i] + k0) : zero_vec;
      rw[i] = (w_src[i] != nullptr && kin) ? *reinterpret_cast<const bf16x8*>(w_src[i] + k0) : zero_vec;
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0.f;

  int wrow[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) wrow[ni] = (EPI == TAAC_EPI_SWIGLU) ? ni * 64 + wn * 32 : wn * 64 + ni * 32;

  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += BK) {
    if (k0 > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < LD; ++i) {
      *reinterpret_cast<bf16x8*>(&sA[lds_off[i]]) = ra[i];
      *reinterpret_cast<bf16x8*>(&sW[lds_off[i]]) = rw[i];
    }
    __syncthreads();
    if (k0 + BK < p.K) fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 wf[2], af[2];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
        wf[ni] = *reinterpret_cast<const bf16x8*>(&sW[(wrow[ni] + l32) * STR + ks * 16 + hh * 8]);
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
        af[mi] = *reinterpret_cast<const bf16x8*>(&sA[(wt * 64 + mi * 32 + l32) * STR + ks * 16 + hh * 8]);
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
          acc[ni][mi] = Mfma16<T>::run(wf[ni], af[mi], acc[ni][mi]);
    }
  }
  store_tile<EPI, T>(p, acc, 1.0f, m0, n0, wt, wn, l32, hh);
}

// ------------------------------------------------------------------------------------------------------------------
// bf16 operands, narrow outputs from a long contraction (128 < N <= 256, K a multiple of 32): the input-gradient
// products of the backward (dy w with K = 2F or 3D, N = D). One workgroup owns 256 tokens x ALL output features, so the
// activations are read from memory exactly once (the 128 x 128 kernel reads them once per feature tile: 0.80 ms against
// 0.57 ms for the library at M = 524 288, K = 2048). Eight wavefronts, 4 token groups of 64 x 2 feature halves of 128:
// per k-step 4 weight fragments and 2 token fragments from LDS feed 8 MFMAs. K is walked in slabs of 32: the slab of
// both operands goes from global memory straight into LDS (16 rows x 64 bytes per transfer instruction, 4 instructions
// per wavefront and slab) into a ring of four 32 KB stages, three slabs ahead (a first version staged 64-wide slabs
// through registers, one slab ahead: the same 0.73 ms, so it is not the latency of the loads that bounds the kernel at
// 3.3-3.5 TB/s; half of the wavefronts' time is spent waiting for the transfers). A transfer cannot pad rows, so the four 16-byte pieces of a row are XOR-swizzled
// by (row / 4) % 4: the 16 lanes of a fragment read hit 16 distinct bank groups. Rows beyond M (or N) repeat the last
// row; their results are not stored.
// ------------------------------------------------------------------------------------------------------------------
constexpr int kWideThreads = 512;
constexpr int kWideTile = 256;
constexpr int kWideSlab = 32;
constexpr int kWideRing = 4;
constexpr int kWideOperandBytes = kWideTile * kWideSlab * 2;   // 16 KB
constexpr int kWideStageBytes = 2 * kWideOperandBytes;         // tokens | weights
constexpr size_t kWideLdsBytes = static_cast<size_t>(kWideRing) * kWideStageBytes;

template <int EPI>
__global__ __launch_bounds__(kWideThreads, 2) void linear_bf16_wide_kernel(const LinearParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t wide_smem[];

  const int64_t m0 = static_cast<int64_t>(blockIdx.x) * kWideTile;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int wt = wave % 4;  // token group of 64
  const int wn = wave / 4;  // feature half of 128
  const int nslabs = p.K / kWideSlab;

  // Transfers of this wavefront: instructions j = 2 * wave, 2 * wave + 1 of both operands; lane -> row 16 j + lane / 4,
  // LDS piece lane % 4, which holds global piece (lane % 4) ^ (row / 4) % 4 of the slab.
  const bf16_t* a_src[2];
  const bf16_t* w_src[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = 16 * (2 * wave + i) + lane / 4;
    const int piece = (lane % 4) ^ ((row >> 2) & 3);
    const int64_t arow = m0 + row < p.M ? m0 + row : p.M - 1;
    const int wrow = row < p.N ? row : p.N - 1;
    a_src[i] = static_cast<const bf16_t*>(p.a) + arow * p.lda + piece * 8;
    w_src[i] = static_cast<const bf16_t*>(p.w) + static_cast<int64_t>(wrow) * p.K + piece * 8;
  }
  // Every workgroup starts its walk over K at a different slab (the sum is the same; its order differs per workgroup,
  // not per run): with all workgroups on the same columns of a matrix whose row pitch is a power of two their requests
  // crowded the same memory channels (0.73 -> 0.69 ms at K = 2048).
  const int rot = static_cast<int>((blockIdx.x * 5u) % static_cast<uint32_t>(nslabs));
  auto stage = [&](int slab) {
    uint8_t* base = wide_smem + (slab % kWideRing) * kWideStageBytes + (2 * wave) * 1024;
    const int turned = slab + rot;
    const int k0 = (turned >= nslabs ? turned - nslabs : turned) * kWideSlab;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      lds_dma16(a_src[i] + k0, base + i * 1024);
      lds_dma16(w_src[i] + k0, base + kWideOperandBytes + i * 1024);
    }
  };
  // Fragment reads: lane (l32, hh) takes piece 2 ks + hh of its row, stored at piece ^ (l32 / 4) % 4.
  const int swz = (l32 >> 2) & 3;
  int piece_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) piece_off[ks] = ((2 * ks + hh) ^ swz) * 16;
  const int a_row_off = (wt * 64 + l32) * (kWideSlab * 2);
  const int w_row_off = kWideOperandBytes + (wn * 128 + l32) * (kWideSlab * 2);

  f32x16 acc[4][2];
#pragma unroll
  for (int ni = 0; ni < 4; ++ni)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0.f;

#pragma unroll
  for (int q = 0; q < kWideRing - 1; ++q)
    if (q < nslabs) stage(q);
  // slab 0 has landed when at most the transfers of slabs 1 and 2 are outstanding
  if (nslabs > 2) vm_wait<8>();
  else if (nslabs > 1) vm_wait<4>();
  else vm_wait<0>();
  __syncthreads();
  for (int s = 0; s < nslabs; ++s) {
    // slot (s + 3) % 4 was last read in slab s - 1, which every wavefront has left
    if (s + kWideRing - 1 < nslabs) stage(s + kWideRing - 1);
    const uint8_t* st = wide_smem + (s % kWideRing) * kWideStageBytes;
#pragma unroll
    for (int ks = 0; ks < kWideSlab / 16; ++ks) {
      bf16x8 wf[4], af[2];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
        af[mi] = *reinterpret_cast<const bf16x8*>(st + a_row_off + mi * 32 * (kWideSlab * 2) + piece_off[ks]);
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
        wf[ni] = *reinterpret_cast<const bf16x8*>(st + w_row_off + ni * 32 * (kWideSlab * 2) + piece_off[ks]);
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
          acc[ni][mi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ni], af[mi], acc[ni][mi], 0, 0, 0);
    }
    if (s + 1 < nslabs) {
      // the transfers of slab s + 1 were issued three slabs ago; behind them are those of slabs s + 2 and s + 3
      if (s + 3 < nslabs) vm_wait<8>();
      else if (s + 2 < nslabs) vm_wait<4>();
      else vm_wait<0>();
      __syncthreads();
    }
  }

  // acc[ni][mi][jq * 4 + e]: feature wn * 128 + ni * 32 + jq * 8 + hh * 4 + e of token wt * 64 + mi * 32 + l32
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int64_t row = m0 + wt * 64 + mi * 32 + l32;
    if (row >= p.M) continue;
    bf16_t* orow = static_cast<bf16_t*>(p.out) + row * p.ldo;
    const bf16_t* rrow = (EPI == TAAC_EPI_RESIDUAL) ? static_cast<const bf16_t*>(p.residual) + row * p.ldo : nullptr;
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) {
#pragma unroll
      for (int jq = 0; jq < 4; ++jq) {
        const int col = wn * 128 + ni * 32 + jq * 8 + hh * 4;
        if (col >= p.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[ni][mi][jq * 4 + e];
        if (p.bias != nullptr) {
          const bf16x4 bv = *reinterpret_cast<const bf16x4*>(static_cast<const bf16_t*>(p.bias) + col);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += static_cast<float>(bv[e]);
        }
        if (EPI == TAAC_EPI_RESIDUAL) {
          const bf16x4 rv = *reinterpret_cast<const bf16x4*>(rrow + col);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += static_cast<float>(rv[e]);
        }
        bf16x4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = static_cast<bf16_t>(v[e]);
        *reinterpret_cast<bf16x4*>(orow + col) = ov;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// fp8 (OCP e4m3fn) operands, per-tensor scales. Activations arrive as bf16 and are quantised while being staged
// (A_FP8 == false), or are already e4m3 bytes (A_FP8 == true).
// ------------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float clamp448(float x) { return __builtin_fminf(__builtin_fmaxf(x, -448.f), 448.f); }

// 8 bf16 -> 8 e4m3 bytes (two dwords), value * inv_scale, saturating, round to nearest even.
__device__ __forceinline__ u32x2 quant8(const bf16x8& v, float inv_scale) {
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = clamp448(static_cast<float>(v[e]) * inv_scale);
  u32x2 r;
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
  r[0] = static_cast<uint32_t>(lo);
  r[1] = static_cast<uint32_t>(hi);
  return r;
}

template <int EPI, bool A_FP8>
__global__ __launch_bounds__(kThreads) void linear_fp8_kernel(const LinearParams p) {
  constexpr int BK = 128;              // bytes == elements per tile row
  constexpr int STR = BK + 16;         // LDS row stride in bytes
  constexpr int CH = BK / 16;          // 16-byte chunks per tile row (8)
  constexpr int LD = kBM * CH / kThreads;  // 4
  __shared__ __attribute__((aligned(16))) uint8_t sA[kBM * STR];
  __shared__ __attribute__((aligned(16))) uint8_t sW[kBN * STR];

  const uint32_t logical = xcd_remap(blockIdx.x, p.total);
  const int nt = static_cast<int>(logical % p.ntiles);
  const int64_t mt = logical / p.ntiles;
  const int64_t m0 = mt * kBM;
  const int n0 = nt * (EPI == TAAC_EPI_SWIGLU ? 64 : kBN);

  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int wt = wave % 2;
  const int wn = wave / 2;

  const float amax_a = fmaxf(*p.amax_a, 1e-12f);
  const float amax_w = fmaxf(*p.amax_w, 1e-12f);
  const float inv_scale_a = 448.0f / amax_a;
  const float dq = (amax_a / 448.0f) * (amax_w / 448.0f);

  const uint8_t* W = static_cast<const uint8_t*>(p.w);
  u32x4 zero4 = {0u, 0u, 0u, 0u};

  int lds_off[LD], col_off[LD];
  int64_t a_row[LD];
  const uint8_t* w_src[LD];
#pragma unroll
  for (int i = 0; i < LD; ++i) {
    const int cidx = tid + kThreads * i;
    const int r = cidx / CH;
    const int c16 = cidx % CH;
    lds_off[i] = r * STR + c16 * 16;
    col_off[i] = c16 * 16;
    a_row[i] = (m0 + r < p.M) ? (m0 + r) : -1;
    w_src[i] = weight_row_ok<EPI>(p, n0, r) ? W + static_cast<int64_t>(weight_row<EPI>(p, n0, r)) * p.K + c16 * 16
                                             : nullptr;
  }

  u32x4 rw[LD];
  u32x4 ra8[LD];         // A_FP8: raw bytes
  bf16x8 ra16[LD][2];    // !A_FP8: 16 bf16 values
  bf16x8 zero_vec;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero_vec[e] = static_cast<bf16_t>(0.f);

  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < LD; ++i) {
      const bool kin = k0 + col_off[i] < p.K;
      rw[i] = (w_src[i] != nullptr && kin) ? *reinterpret_cast<const u32x4*>(w_src[i] + k0) : zero4;
      if (A_FP8) {
        const uint8_t* A = static_cast<const uint8_t*>(p.a);
        ra8[i] = (a_row[i] >= 0 && kin) ? *reinterpret_cast<const u32x4*>(A + a_row[i] * p.lda + k0 + col_off[i])
                                        : zero4;
      } else {
        const bf16_t* A = static_cast<const bf16_t*>(p.a);
        if (a_row[i] >= 0 && kin) {
          const bf16x8* src = reinterpret_cast<const bf16x8*>(A + a_row[i] * p.lda + k0 + col_off[i]);
          ra16[i][0] = src[0];
          ra16[i][1] = src[1];
        } else {
          ra16[i][0] = zero_vec;
          ra16[i][1] = zero_vec;
        }
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[ni][mi][j] = 0.f;

  int wrow[2];
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) wrow[ni] = (EPI == TAAC_EPI_SWIGLU) ? ni * 64 + wn * 32 : wn * 64 + ni * 32;

  constexpr int kScaleOne = 127;  // E8M0 exponent of 1.0 for the block-scale operands of the f8f6f4 MFMA

  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += BK) {
    if (k0 > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < LD; ++i) {
      *reinterpret_cast<u32x4*>(&sW[lds_off[i]]) = rw[i];
      if (A_FP8) {
        *reinterpret_cast<u32x4*>(&sA[lds_off[i]]) = ra8[i];
      } else {
        const u32x2 q0 = quant8(ra16[i][0], inv_scale_a);
        const u32x2 q1 = quant8(ra16[i][1], inv_scale_a);
        u32x4 q = {q0[0], q0[1], q1[0], q1[1]};
        *reinterpret_cast<u32x4*>(&sA[lds_off[i]]) = q;
      }
    }
    __syncthreads();
    if (k0 + BK < p.K) fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < BK / 64; ++ks) {
      i32x8 wf[2], af[2];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const u32x4* src = reinterpret_cast<const u32x4*>(&sW[(wrow[ni] + l32) * STR + ks * 64 + hh * 32]);
        const u32x4 lo = src[0], hi = src[1];
        wf[ni] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) {
        const u32x4* src = reinterpret_cast<const u32x4*>(&sA[(wt * 64 + mi * 32 + l32) * STR + ks * 64 + hh * 32]);
        const u32x4 lo = src[0], hi = src[1];
        af[mi] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
          acc[ni][mi] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[ni], af[mi], acc[ni][mi], 0, 0, 0, kScaleOne,
                                                                        0, kScaleOne);
    }
  }
  store_tile<EPI>(p, acc, dq, m0, n0, wt, wn, l32, hh);
}

int validate_common(const char* name, const void* a, const void* w, const void* out, const void* residual,
                    int64_t lda, int64_t ldo, int64_t M, int32_t N, int32_t K, int epilogue, int k_mult) {
  if (M < 0 || N <= 0 || K <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, N and K > 0", name);
  if (epilogue != TAAC_EPI_NONE && epilogue != TAAC_EPI_RESIDUAL && epilogue != TAAC_EPI_SWIGLU)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown epilogue %d", name, epilogue);
  if (K % k_mult != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: K=%d must be a multiple of %d", name, K, k_mult);
  if (epilogue == TAAC_EPI_SWIGLU) {
    if (N % 16 != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: SwiGLU needs N=%d to be a multiple of 16", name, N);
  } else if (N % 8 != 0) {
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d must be a multiple of 8", name, N);
  }
  const int64_t n_out = epilogue == TAAC_EPI_SWIGLU ? N / 2 : N;
  if (lda < K || ldo < n_out || lda % 8 != 0 || ldo % 8 != 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (M == 0) return TAAC_OK;
  if (!a || !w || !out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (epilogue == TAAC_EPI_RESIDUAL && !residual)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: residual epilogue without a residual tensor", name);
  if (!aligned16(a) || !aligned16(w) || !aligned16(out) || (residual && !aligned16(residual)))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  return TAAC_OK;
}

int fill_params(const char* name, LinearParams& p, int64_t M, int32_t N, int epilogue) {
  p.F = N / 2;
  const int64_t mtiles = (M + kBM - 1) / kBM;
  const int64_t ntiles = epilogue == TAAC_EPI_SWIGLU ? (p.F + 63) / 64 : (N + kBN - 1) / kBN;
  const int64_t total = mtiles * ntiles;
  if (total > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  p.ntiles = static_cast<uint32_t>(ntiles);
  p.total = static_cast<uint32_t>(total);
  return TAAC_OK;
}

}  // namespace
}  // namespace taac

extern "C" int taac_linear_bf16(const void* a, int64_t lda, const void* w, const void* bias, const void* residual,
                                void* out, int64_t ldo, int64_t M, int32_t N, int32_t K, int epilogue, int gate_first,
                                void* stream) {
  using namespace taac;
  const char* name = "taac_linear_bf16";
  int rc = validate_common(name, a, w, out, residual, lda, ldo, M, N, K, epilogue, 8);
  if (rc != TAAC_OK || M == 0) return rc;
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 7u))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: bias must be 8-byte aligned", name);
  LinearParams p{};
  p.a = a;
  p.w = w;
  p.bias = bias;
  p.residual = residual;
  p.out = out;
  p.lda = lda;
  p.ldo = ldo;
  p.M = M;
  p.N = N;
  p.K = K;
  p.gate_first = gate_first ? 1 : 0;
  rc = fill_params(name, p, M, N, epilogue);
  if (rc != TAAC_OK) return rc;
  hipStream_t s = as_stream(stream);
  if (epilogue != TAAC_EPI_SWIGLU && N > 128 && N <= kWideTile && K >= 512 && K % kWideSlab == 0 && M >= 1024) {
    // long contraction into a narrow output: one workgroup per 256 tokens with all output features
    const int64_t blocks = (M + kWideTile - 1) / kWideTile;
    if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
    const void* kernel = epilogue == TAAC_EPI_NONE ? reinterpret_cast<const void*>(linear_bf16_wide_kernel<TAAC_EPI_NONE>)
                                                   : reinterpret_cast<const void*>(linear_bf16_wide_kernel<TAAC_EPI_RESIDUAL>);
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kWideLdsBytes)) != hipSuccess)
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, kWideLdsBytes);
    if (epilogue == TAAC_EPI_NONE)
      hipLaunchKernelGGL((linear_bf16_wide_kernel<TAAC_EPI_NONE>), dim3(static_cast<uint32_t>(blocks)), dim3(kWideThreads),
                         kWideLdsBytes, s, p);
    else
      hipLaunchKernelGGL((linear_bf16_wide_kernel<TAAC_EPI_RESIDUAL>), dim3(static_cast<uint32_t>(blocks)),
                         dim3(kWideThreads), kWideLdsBytes, s, p);
    return check_launch(name);
  }
  switch (epilogue) {
    case TAAC_EPI_NONE:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_NONE>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
    case TAAC_EPI_RESIDUAL:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_RESIDUAL>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
    default:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_SWIGLU>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
  }
  return check_launch(name);
}

extern "C" int taac_linear_f16(const void* a, int64_t lda, const void* w, const void* bias, const void* residual,
                               void* out, int64_t ldo, int64_t M, int32_t N, int32_t K, int epilogue, int gate_first,
                               void* stream) {
  using namespace taac;
  const char* name = "taac_linear_f16";
  int rc = validate_common(name, a, w, out, residual, lda, ldo, M, N, K, epilogue, 8);
  if (rc != TAAC_OK || M == 0) return rc;
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 7u))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: bias must be 8-byte aligned", name);
  LinearParams p{};
  p.a = a;
  p.w = w;
  p.bias = bias;
  p.residual = residual;
  p.out = out;
  p.lda = lda;
  p.ldo = ldo;
  p.M = M;
  p.N = N;
  p.K = K;
  p.gate_first = gate_first ? 1 : 0;
  rc = fill_params(name, p, M, N, epilogue);
  if (rc != TAAC_OK) return rc;
  hipStream_t s = as_stream(stream);
  switch (epilogue) {
    case TAAC_EPI_NONE:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_NONE, f16_t>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
    case TAAC_EPI_RESIDUAL:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_RESIDUAL, f16_t>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
    default:
      hipLaunchKernelGGL((linear_bf16_kernel<TAAC_EPI_SWIGLU, f16_t>), dim3(p.total), dim3(kThreads), 0, s, p);
      break;
  }
  return check_launch(name);
}

extern "C" int taac_linear_fp8(const void* a, int a_is_fp8, int64_t lda, const void* w, const float* amax_a,
                               const float* amax_w, const void* bias, const void* residual, void* out, int64_t ldo,
                               int64_t M, int32_t N, int32_t K, int epilogue, int gate_first, void* stream) {
  using namespace taac;
  const char* name = "taac_linear_fp8";
  int rc = validate_common(name, a, w, out, residual, lda, ldo, M, N, K, epilogue, 16);
  if (rc != TAAC_OK || M == 0) return rc;
  if (!amax_a || !amax_w) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null amax pointer", name);
  if (a_is_fp8 && lda % 16 != 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: fp8 activations need a row stride that is a multiple of 16", name);
  if (bias && (reinterpret_cast<uintptr_t>(bias) & 7u))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: bias must be 8-byte aligned", name);
  LinearParams p{};
  p.a = a;
  p.w = w;
  p.bias = bias;
  p.residual = residual;
  p.out = out;
  p.amax_a = amax_a;
  p.amax_w = amax_w;
  p.lda = lda;
  p.ldo = ldo;
  p.M = M;
  p.N = N;
  p.K = K;
  p.gate_first = gate_first ? 1 : 0;
  rc = fill_params(name, p, M, N, epilogue);
  if (rc != TAAC_OK) return rc;
  hipStream_t s = as_stream(stream);
  rc = launch_linear_fp8_ts(a, a_is_fp8, lda, w, amax_a, amax_w, bias, residual, out, ldo, M, N, K, epilogue, gate_first,
                            s, name);
  if (rc <= 0) return rc;  // launched (or failed) on the token-stationary path
#define TAAC_FP8_LAUNCH(EPI)                                                                                   \
  if (a_is_fp8)                                                                                                \
    hipLaunchKernelGGL((linear_fp8_kernel<EPI, true>), dim3(p.total), dim3(kThreads), 0, s, p);               \
  else                                                                                                         \
    hipLaunchKernelGGL((linear_fp8_kernel<EPI, false>), dim3(p.total), dim3(kThreads), 0, s, p);
  switch (epilogue) {
    case TAAC_EPI_NONE: TAAC_FP8_LAUNCH(TAAC_EPI_NONE) break;
    case TAAC_EPI_RESIDUAL: TAAC_FP8_LAUNCH(TAAC_EPI_RESIDUAL) break;
    default: TAAC_FP8_LAUNCH(TAAC_EPI_SWIGLU) break;
  }
#undef TAAC_FP8_LAUNCH
  return check_launch(name);
}
