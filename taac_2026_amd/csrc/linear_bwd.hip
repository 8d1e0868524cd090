// Backward pieces of the dense layers (gfx950): the weight gradient of a linear layer as a product over the tokens, the
// column sums for the bias gradient, and the elementwise backward of the SiLU gate.
//
//   taac_linear_wgrad : dW[n, k] = sum_m dy[m, n] * a[m, k],  db[n] = sum_m dy[m, n]
//   taac_swiglu_bwd   : hidden = silu(g) * u,  dg = dhidden * u * silu'(g),  du = dhidden * silu(g)
//
// The reference trains its dense layers through torch autograd of nn.Linear / F.silu (experiments/symbiosis/backbone.py:
// 11-21, 24-48); these are the two products of that backward that are not themselves a forward-shaped linear layer (the
// input gradient dy W is one, with the transposed weight).
//
// Weight gradient: both operands are [tokens, features] row-major, and the MFMA needs, per lane, eight consecutive tokens
// of one feature from each - a transposed read. HBM-bound (the operands are read, the result is tiny), so the kernel is
// built to read them as few times as possible and to keep loads in flight: a workgroup of eight wavefronts owns a
// 256 x 256 tile of dW (128 accumulator registers per lane) over its share of the tokens, so with K = 256 dy is read once
// and a once per 256 output features; 64-token chunks of both 256-feature slabs go through registers into one of two LDS
// buffers (row-major, rows padded to 544 bytes: the four rows and four 8-byte pieces a 16-lane group touches fall on
// distinct banks) while the chunk before is multiplied, one barrier per chunk, and both fragments are read with
// ds_read_b64_tr_b16. Shapes below 256 in either dimension keep the 128 x 128 tile of four wavefronts. The token range is
// split over workgroups; every split writes its fp32 partial tile, and a second kernel adds the splits in a fixed order,
// so the gradient is bit-reproducible.

#include <hip/hip_runtime.h>
#include <math.h>

#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kThreads = 256;
constexpr int kTile = 128;      // features of dy / of a per workgroup tile
constexpr int kChunk = 32;      // tokens per staged chunk
constexpr int kRowBytes = kTile * 2 + 32;  // padded LDS row
constexpr int kMaxSplits = 256;

// Stage rows [m0, m0 + 32) x columns [c0, c0 + 128) of src (bf16, row stride ld) into dst; out-of-range pieces are zeros.
__device__ __forceinline__ void stage_chunk(const bf16_t* __restrict__ src, int64_t ld, int64_t m0, int64_t m_end, int c0,
                                            int cols, uint8_t* dst, int tid) {
#pragma unroll
  for (int i = 0; i < kChunk * (kTile / 8) / kThreads; ++i) {
    const int idx = tid + i * kThreads;
    const int row = idx / (kTile / 8), piece = idx % (kTile / 8);
    const int64_t m = m0 + row;
    const int c = c0 + piece * 8;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (m < m_end && c < cols) v = *reinterpret_cast<const u32x4*>(src + m * ld + c);
    *reinterpret_cast<u32x4*>(dst + row * kRowBytes + piece * 16) = v;
  }
}

// grid = (tiles of N x tiles of K, splits). partial: [splits][N][K] fp32.
__global__ __launch_bounds__(kThreads) void wgrad_partial_kernel(const bf16_t* __restrict__ dy, int64_t ldy,
                                                                 const bf16_t* __restrict__ a, int64_t lda,
                                                                 float* __restrict__ partial, int64_t M, int N, int K,
                                                                 int64_t rows_per_split) {
  __shared__ __attribute__((aligned(16))) uint8_t smem[2 * kChunk * kRowBytes];
  uint8_t* sA = smem;                       // dy slab
  uint8_t* sB = smem + kChunk * kRowBytes;  // activation slab
  const int tiles_k = (K + kTile - 1) / kTile;
  const int n0 = (blockIdx.x / tiles_k) * kTile, k0 = (blockIdx.x % tiles_k) * kTile;
  const int64_t m_begin = static_cast<int64_t>(blockIdx.y) * rows_per_split;
  const int64_t m_end = m_begin + rows_per_split < M ? m_begin + rows_per_split : M;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int wn = wave / 2, wk = wave % 2;  // the wavefront's 64 x 64 block of the tile
  // transposed read: lane r of a 16-lane group g points at token t0 + r / 4, features f0 + 4 * (r % 4) .. + 3 and receives
  // tokens t0 .. t0 + 3 of feature f0 + r; group g covers features 16 * (g % 2) .. + 15 and the token half g / 2
  const int g = lane / 16, r = lane % 16;
  const uint32_t lane_off = static_cast<uint32_t>((8 * (g / 2) + r / 4) * kRowBytes + (16 * (g % 2) + 4 * (r % 4)) * 2);
  const uint32_t a_addr = lds_offset(sA) + lane_off + wn * 64 * 2;
  const uint32_t b_addr = lds_offset(sB) + lane_off + wk * 64 * 2;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  for (int64_t m0 = m_begin; m0 < m_end; m0 += kChunk) {
    __syncthreads();  // everyone is done reading the previous chunk
    stage_chunk(dy, ldy, m0, m_end, n0, N, sA, tid);
    stage_chunk(a, lda, m0, m_end, k0, K, sB, tid);
    __syncthreads();
    static_for<kChunk / 16>([&](auto ks_tag) {
      constexpr int ks = decltype(ks_tag)::value;
      u32x2 fa[2][2], fb[2][2];
      static_for<2>([&](auto t_tag) {
        constexpr int t = decltype(t_tag)::value;
        lds_read_tr16<(ks * 16) * kRowBytes + t * 64>(fa[t][0], a_addr);
        lds_read_tr16<(ks * 16 + 4) * kRowBytes + t * 64>(fa[t][1], a_addr);
        lds_read_tr16<(ks * 16) * kRowBytes + t * 64>(fb[t][0], b_addr);
        lds_read_tr16<(ks * 16 + 4) * kRowBytes + t * 64>(fb[t][1], b_addr);
      });
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[1][0]), "+v"(fa[1][1]) : : "memory");
      asm volatile("" : "+v"(fb[0][0]), "+v"(fb[0][1]), "+v"(fb[1][0]), "+v"(fb[1][1]));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x4 abits = {fa[i][0][0], fa[i][0][1], fa[i][1][0], fa[i][1][1]};
          const u32x4 bbits = {fb[j][0][0], fb[j][0][1], fb[j][1][0], fb[j][1][1]};
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, abits),
                                                              __builtin_bit_cast(bf16x8, bbits), acc[i][j], 0, 0, 0);
        }
    });
  }
  // accumulator register e of a lane: row (e / 4) * 8 + (lane / 32) * 4 + e % 4 of the 32 x 32 tile, column lane % 32
  float* out = partial + static_cast<int64_t>(blockIdx.y) * N * K;
  const int l32 = lane % 32, hh = lane / 32;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = k0 + wk * 64 + j * 32 + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = n0 + wn * 64 + i * 32 + (e / 4) * 8 + hh * 4 + (e % 4);
        if (row < N && col < K) out[static_cast<int64_t>(row) * K + col] = acc[i][j][e];
      }
    }
}

// ---- 256 x 256 tile, eight wavefronts, chunks of 64 tokens, registers -> double-buffered LDS --------------------------
constexpr int kBigThreads = 512;
constexpr int kBigTile = 256;
constexpr int kBigChunk = 64;
constexpr int kBigRowBytes = kBigTile * 2 + 32;
constexpr int kBigPieces = kBigChunk * (kBigTile / 8) / kBigThreads;  // 16-byte pieces per thread, operand and chunk

__device__ __forceinline__ void big_fetch(const bf16_t* __restrict__ src, int64_t ld, int64_t m0, int64_t m_end, int c0,
                                          int cols, int tid, u32x4 (&v)[kBigPieces]) {
#pragma unroll
  for (int i = 0; i < kBigPieces; ++i) {
    const int idx = tid + i * kBigThreads;
    const int row = idx / (kBigTile / 8), piece = idx % (kBigTile / 8);
    const int64_t m = m0 + row;
    const int c = c0 + piece * 8;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    v[i] = (m < m_end && c < cols) ? *reinterpret_cast<const u32x4*>(src + m * ld + c) : zero;
  }
}
__device__ __forceinline__ void big_commit(uint8_t* dst, int tid, const u32x4 (&v)[kBigPieces]) {
#pragma unroll
  for (int i = 0; i < kBigPieces; ++i) {
    const int idx = tid + i * kBigThreads;
    *reinterpret_cast<u32x4*>(dst + (idx / (kBigTile / 8)) * kBigRowBytes + (idx % (kBigTile / 8)) * 16) = v[i];
  }
}

// grid = (tiles of N x tiles of K, splits). partial: [splits][N][K] fp32.
__global__ __launch_bounds__(kBigThreads, 2) void wgrad_partial_big_kernel(const bf16_t* __restrict__ dy, int64_t ldy,
                                                                          const bf16_t* __restrict__ a, int64_t lda,
                                                                          float* __restrict__ partial,
                                                                          float* __restrict__ partial_bias, int64_t M,
                                                                          int N, int K, int64_t rows_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint8_t big_smem[];
  constexpr int kSlab = kBigChunk * kBigRowBytes;  // one operand of one chunk
  const int tiles_k = (K + kBigTile - 1) / kBigTile;
  const int n0 = (blockIdx.x / tiles_k) * kBigTile, k0 = (blockIdx.x % tiles_k) * kBigTile;
  const int64_t m_begin = static_cast<int64_t>(blockIdx.y) * rows_per_split;
  const int64_t m_end = m_begin + rows_per_split < M ? m_begin + rows_per_split : M;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
  const int wn = wave / 4, wk = wave % 4;  // the wavefront's 128 (n) x 64 (k) block of the tile
  const int g = lane / 16, r = lane % 16;
  const uint32_t lane_off = static_cast<uint32_t>((8 * (g / 2) + r / 4) * kBigRowBytes + (16 * (g % 2) + 4 * (r % 4)) * 2);
  const uint32_t a_lane = lane_off + wn * 128 * 2;
  const uint32_t b_lane = kSlab + lane_off + wk * 64 * 2;

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  u32x4 va[kBigPieces], vb[kBigPieces];
  if (m_begin < m_end) {
    big_fetch(dy, ldy, m_begin, m_end, n0, N, tid, va);
    big_fetch(a, lda, m_begin, m_end, k0, K, tid, vb);
  }
  // Bias gradient (column sums of dy) on the way: the workgroups of the first K tile add up the dy pieces they stage -
  // a thread always holds the same eight columns, of rows tid / 32 + 16 i - and combine the 16 row groups at the end.
  const bool with_bias = partial_bias != nullptr && k0 == 0;
  float csum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  int buf = 0;
  for (int64_t m0 = m_begin; m0 < m_end; m0 += kBigChunk) {
    // the buffer written now was last read two chunks ago; the barrier of the chunk in between lies behind those reads
    uint8_t* stage = big_smem + buf * (2 * kSlab);
    if (with_bias) {
#pragma unroll
      for (int i = 0; i < kBigPieces; ++i)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          csum[2 * w] += __uint_as_float(va[i][w] << 16);
          csum[2 * w + 1] += __uint_as_float(va[i][w] & 0xffff0000u);
        }
    }
    big_commit(stage, tid, va);
    big_commit(stage + kSlab, tid, vb);
    if (m0 + kBigChunk < m_end) {
      big_fetch(dy, ldy, m0 + kBigChunk, m_end, n0, N, tid, va);
      big_fetch(a, lda, m0 + kBigChunk, m_end, k0, K, tid, vb);
    }
    __syncthreads();
    const uint32_t base = lds_offset(stage);
    static_for<kBigChunk / 16>([&](auto ks_tag) {
      constexpr int ks = decltype(ks_tag)::value;
      u32x2 fa[4][2], fb[2][2];
      static_for<4>([&](auto t_tag) {
        constexpr int t = decltype(t_tag)::value;
        lds_read_tr16<(ks * 16) * kBigRowBytes + t * 64>(fa[t][0], base + a_lane);
        lds_read_tr16<(ks * 16 + 4) * kBigRowBytes + t * 64>(fa[t][1], base + a_lane);
      });
      static_for<2>([&](auto t_tag) {
        constexpr int t = decltype(t_tag)::value;
        lds_read_tr16<(ks * 16) * kBigRowBytes + t * 64>(fb[t][0], base + b_lane);
        lds_read_tr16<(ks * 16 + 4) * kBigRowBytes + t * 64>(fb[t][1], base + b_lane);
      });
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[1][0]), "+v"(fa[1][1]), "+v"(fa[2][0]), "+v"(fa[2][1]),
                     "+v"(fa[3][0]), "+v"(fa[3][1])
                   :
                   : "memory");
      asm volatile("" : "+v"(fb[0][0]), "+v"(fb[0][1]), "+v"(fb[1][0]), "+v"(fb[1][1]));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x4 abits = {fa[i][0][0], fa[i][0][1], fa[i][1][0], fa[i][1][1]};
          const u32x4 bbits = {fb[j][0][0], fb[j][0][1], fb[j][1][0], fb[j][1][1]};
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, abits),
                                                              __builtin_bit_cast(bf16x8, bbits), acc[i][j], 0, 0, 0);
        }
    });
    buf ^= 1;
  }
  float* out = partial + static_cast<int64_t>(blockIdx.y) * N * K;
  const int l32 = lane % 32, hh = lane / 32;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = k0 + wk * 64 + j * 32 + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = n0 + wn * 128 + i * 32 + (e / 4) * 8 + hh * 4 + (e % 4);
        if (row < N && col < K) out[static_cast<int64_t>(row) * K + col] = acc[i][j][e];
      }
    }
  if (with_bias) {
    __syncthreads();  // every wavefront is done with the chunk buffers
    float* red = reinterpret_cast<float*>(big_smem);  // [16 row groups][256 columns]
#pragma unroll
    for (int e = 0; e < 8; ++e) red[(tid / 32) * kBigTile + (tid % 32) * 8 + e] = csum[e];
    __syncthreads();
    if (tid < kBigTile && n0 + tid < N) {
      float sum = 0.f;
#pragma unroll
      for (int rg = 0; rg < kBigThreads / 32; ++rg) sum += red[rg * kBigTile + tid];
      partial_bias[static_cast<int64_t>(blockIdx.y) * N + n0 + tid] = sum;
    }
  }
}

// out[i] = sum over the splits of partial[s][i], in split order; one rounding to the output type.
template <typename TOut>
__global__ __launch_bounds__(kThreads) void reduce_splits_kernel(const float* __restrict__ partial, TOut* __restrict__ out,
                                                                 int64_t n, int splits) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int k = 0; k < splits; ++k) s += partial[static_cast<int64_t>(k) * n + i];
  out[i] = static_cast<TOut>(s);
}

// partial[split][c] = sum over the split's rows of dy[m][c]. A workgroup covers 256 columns: thread (column group
// tid % 32 of eight columns, row lane tid / 32) adds every eighth row; the eight row lanes are combined through LDS in a
// fixed order.
__global__ __launch_bounds__(kThreads) void colsum_partial_kernel(const bf16_t* __restrict__ dy, int64_t ldy,
                                                                  float* __restrict__ partial, int64_t M, int N,
                                                                  int64_t rows_per_split) {
  __shared__ float red[kThreads / 32][256];
  const int64_t m_begin = static_cast<int64_t>(blockIdx.y) * rows_per_split;
  const int64_t m_end = m_begin + rows_per_split < M ? m_begin + rows_per_split : M;
  const int tid = threadIdx.x;
  const int c = blockIdx.x * 256 + (tid % 32) * 8;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (c < N) {
    for (int64_t m = m_begin + tid / 32; m < m_end; m += kThreads / 32) {
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(dy + m * ldy + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] += static_cast<float>(v[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[tid / 32][(tid % 32) * 8 + e] = s[e];
  __syncthreads();
  const int col = blockIdx.x * 256 + tid;
  if (col < N) {
    float sum = 0.f;
#pragma unroll
    for (int rl = 0; rl < kThreads / 32; ++rl) sum += red[rl][tid];
    partial[static_cast<int64_t>(blockIdx.y) * N + col] = sum;
  }
}

int splits_for(int64_t M) {
  int64_t s = (M + 2047) / 2048;
  if (s < 1) s = 1;
  if (s > kMaxSplits) s = kMaxSplits;
  return static_cast<int>(s);
}

// gu: [M, 2F] pre-activations (first half g, second half u); dh: [M, F]. gate_first: hidden = silu(g) * u, else g * silu(u).
__global__ __launch_bounds__(kThreads) void swiglu_bwd_kernel(const bf16_t* __restrict__ gu, int64_t ldgu,
                                                              const bf16_t* __restrict__ dh, int64_t lddh,
                                                              bf16_t* __restrict__ dgu, int64_t lddgu,
                                                              bf16_t* __restrict__ hidden, int64_t ldh, int64_t M, int F,
                                                              int gate_first) {
  const int pieces = F / 8;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= M * pieces) return;
  const int64_t m = idx / pieces;
  const int c = static_cast<int>(idx % pieces) * 8;
  const bf16x8 gv = *reinterpret_cast<const bf16x8*>(gu + m * ldgu + c);
  const bf16x8 uv = *reinterpret_cast<const bf16x8*>(gu + m * ldgu + F + c);
  bf16x8 dv;
#pragma unroll
  for (int e = 0; e < 8; ++e) dv[e] = static_cast<bf16_t>(0.f);
  if (dh != nullptr) dv = *reinterpret_cast<const bf16x8*>(dh + m * lddh + c);
  bf16x8 dg, du, hv;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // act: the operand that goes through SiLU; lin: the one that multiplies it
    const float act = static_cast<float>(gate_first ? gv[e] : uv[e]);
    const float lin = static_cast<float>(gate_first ? uv[e] : gv[e]);
    const float d = static_cast<float>(dv[e]);
    const float sig = 1.f / (1.f + __expf(-act));
    const float silu = act * sig;
    const float dact = d * lin * (sig * (1.f + act * (1.f - sig)));
    const float dlin = d * silu;
    hv[e] = static_cast<bf16_t>(silu * lin);
    dg[e] = static_cast<bf16_t>(gate_first ? dact : dlin);
    du[e] = static_cast<bf16_t>(gate_first ? dlin : dact);
  }
  if (dgu != nullptr) {
    *reinterpret_cast<bf16x8*>(dgu + m * lddgu + c) = dg;
    *reinterpret_cast<bf16x8*>(dgu + m * lddgu + F + c) = du;
  }
  if (hidden != nullptr) *reinterpret_cast<bf16x8*>(hidden + m * ldh + c) = hv;
}

}  // namespace
}  // namespace taac

extern "C" int64_t taac_linear_wgrad_workspace_floats(int64_t M, int32_t N, int32_t K) {
  if (M < 0 || N <= 0 || K <= 0) return -1;
  return static_cast<int64_t>(taac::splits_for(M)) * N * (static_cast<int64_t>(K) + 1);
}

extern "C" int taac_linear_wgrad(const void* dy, int64_t ldy, const void* a, int64_t lda, void* dw, void* db,
                                 float* workspace, int64_t workspace_floats, int64_t M, int32_t N, int32_t K, int out_dtype,
                                 void* stream) {
  using namespace taac;
  const char* name = "taac_linear_wgrad";
  if (M < 0 || N <= 0 || K <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, N and K > 0", name);
  if (N % 8 != 0 || K % 8 != 0 || ldy % 8 != 0 || lda % 8 != 0 || ldy < N || lda < K)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: N, K and the row strides must be multiples of 8 and cover a row", name);
  if (out_dtype != TAAC_BF16 && out_dtype != TAAC_F32)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: out_dtype must be bf16 or fp32 (got %d)", name, out_dtype);
  if (!dw || (M > 0 && (!dy || !a))) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!aligned16(dy) || !aligned16(a)) return set_error(TAAC_ERR_UNSUPPORTED, "%s: dy and a must be 16-byte aligned", name);
  const int64_t need = taac_linear_wgrad_workspace_floats(M, N, K);
  if (!workspace || workspace_floats < need)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: workspace must hold %lld floats", name, (long long)need);
  hipStream_t s = as_stream(stream);
  // Large shapes: 256 x 256 tiles, and about one workgroup per compute unit in all (a workgroup fills one with its LDS).
  const bool big = N >= kBigTile && K >= kBigTile && M >= 4 * kBigChunk;
  int splits = splits_for(M);
  int tiles = ((N + kTile - 1) / kTile) * ((K + kTile - 1) / kTile);
  if (big) {
    tiles = ((N + kBigTile - 1) / kBigTile) * ((K + kBigTile - 1) / kBigTile);
    const int cus = compute_units();
    const int want = cus > tiles ? cus / tiles : 1;
    if (want < splits) splits = want;
  }
  const int chunk = big ? kBigChunk : kChunk;
  const int64_t rows_per_split = ((M + splits - 1) / splits + chunk - 1) / chunk * chunk;
  const int64_t nk = static_cast<int64_t>(N) * K;
  float* part_w = workspace;
  float* part_b = workspace + static_cast<int64_t>(splits) * nk;
  if (big) {
    const size_t lds = 2 * 2 * static_cast<size_t>(kBigChunk) * kBigRowBytes;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(wgrad_partial_big_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess)
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds);
    hipLaunchKernelGGL(wgrad_partial_big_kernel, dim3(tiles, splits), dim3(kBigThreads), lds, s,
                       static_cast<const bf16_t*>(dy), ldy, static_cast<const bf16_t*>(a), lda, part_w,
                       db != nullptr ? part_b : nullptr, M, N, K, rows_per_split);
  } else {
    hipLaunchKernelGGL(wgrad_partial_kernel, dim3(tiles, splits), dim3(kThreads), 0, s, static_cast<const bf16_t*>(dy), ldy,
                       static_cast<const bf16_t*>(a), lda, part_w, M, N, K, rows_per_split);
  }
  const uint32_t blocks = static_cast<uint32_t>((nk + kThreads - 1) / kThreads);
  if (out_dtype == TAAC_BF16)
    hipLaunchKernelGGL(reduce_splits_kernel<bf16_t>, dim3(blocks), dim3(kThreads), 0, s, part_w, static_cast<bf16_t*>(dw), nk,
                       splits);
  else
    hipLaunchKernelGGL(reduce_splits_kernel<float>, dim3(blocks), dim3(kThreads), 0, s, part_w, static_cast<float*>(dw), nk,
                       splits);
  if (db != nullptr) {
    if (!big)  // the large-tile kernel has written the partial column sums itself
      hipLaunchKernelGGL(colsum_partial_kernel, dim3((N + 255) / 256, splits), dim3(kThreads), 0, s,
                         static_cast<const bf16_t*>(dy), ldy, part_b, M, N, rows_per_split);
    const uint32_t bblocks = static_cast<uint32_t>((N + kThreads - 1) / kThreads);
    if (out_dtype == TAAC_BF16)
      hipLaunchKernelGGL(reduce_splits_kernel<bf16_t>, dim3(bblocks), dim3(kThreads), 0, s, part_b, static_cast<bf16_t*>(db),
                         static_cast<int64_t>(N), splits);
    else
      hipLaunchKernelGGL(reduce_splits_kernel<float>, dim3(bblocks), dim3(kThreads), 0, s, part_b, static_cast<float*>(db),
                         static_cast<int64_t>(N), splits);
  }
  return check_launch(name);
}

extern "C" int taac_swiglu_bwd(const void* gu, int64_t ldgu, const void* dhidden, int64_t lddh, void* dgu, int64_t lddgu,
                               void* hidden, int64_t ldh, int64_t M, int32_t F, int gate_first, void* stream) {
  using namespace taac;
  const char* name = "taac_swiglu_bwd";
  if (M < 0 || F <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0 and F > 0", name);
  if (F % 8 != 0 || ldgu % 8 != 0 || ldgu < 2 * F || (dhidden && (lddh % 8 != 0 || lddh < F)) ||
      (dgu && (lddgu % 8 != 0 || lddgu < 2 * F)) || (hidden && (ldh % 8 != 0 || ldh < F)))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: F and the row strides must be multiples of 8 and cover a row", name);
  if (M == 0) return TAAC_OK;
  if (!gu || (!dgu && !hidden)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (dgu && !dhidden) return set_error(TAAC_ERR_INVALID_VALUE, "%s: dgu needs dhidden", name);
  if (!aligned16(gu) || !aligned16(dhidden) || !aligned16(dgu) || !aligned16(hidden))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int64_t work = M * (F / 8);
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(static_cast<uint32_t>((work + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     as_stream(stream), static_cast<const bf16_t*>(gu), ldgu, static_cast<const bf16_t*>(dhidden), lddh,
                     static_cast<bf16_t*>(dgu), lddgu, static_cast<bf16_t*>(hidden), ldh, M, F, gate_first ? 1 : 0);
  return check_launch(name);
}
