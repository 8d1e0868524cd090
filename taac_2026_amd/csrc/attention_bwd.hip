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
// second product of each pair consumes those values as a B operand; the streamed A operand for it is staged
// transposed with its 16-row groups permuted to that register order (vt_pos16).
#include <math.h>

#include "common.h"

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

// Position of row k (0..15 inside a 16-row group) in a transposed, permuted LDS row: accumulator order.
__device__ __forceinline__ int vt_pos16(int k) { return ((k >> 2) & 1) * 8 + (k >> 3) * 4 + (k & 3); }

// Staging of a chunk of streamed rows is split into a register fetch and an LDS commit, so that the global loads of
// chunk c + 1 are in flight while chunk c is being consumed.
//
// RowStager: rows [row0, row0 + kChunk) of a [rows, d] matrix (row stride `stride`) -> dst[row][DP + 8]; rows at or
// beyond row_end and features at or beyond d are zeros.
template <typename T, int DP>
struct RowStager {
  typedef typename Vec8<T>::type vec_t;
  static constexpr int C8 = DP / 8, STR = DP + 8;
  static constexpr int N = (kChunk * C8 + kThreads - 1) / kThreads;
  vec_t reg[N];
  __device__ __forceinline__ void fetch(const T* __restrict__ base, int64_t stride, int row0, int row_end, int d, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + i * kThreads;
      const int row = row0 + idx / C8, c8 = idx % C8;
      if (idx < kChunk * C8 && row < row_end && c8 * 8 < d) {
        reg[i] = *reinterpret_cast<const vec_t*>(base + row * stride + c8 * 8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) reg[i][e] = static_cast<T>(0.f);
      }
    }
  }
  __device__ __forceinline__ void commit(T* __restrict__ dst, int tid) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + i * kThreads;
      if (idx < kChunk * C8) *reinterpret_cast<vec_t*>(&dst[(idx / C8) * STR + (idx % C8) * 8]) = reg[i];
    }
  }
};

// TransStager: the same rows transposed, dst[feature][pos(row)] with row stride kChunk + 8, the rows of every 16-row
// group in accumulator order, two neighbouring rows per 32-bit store.
template <typename T, int DP>
struct TransStager {
  typedef typename Vec8<T>::type vec_t;
  static constexpr int C8 = DP / 8, STR = kChunk + 8;
  static constexpr int N = ((kChunk / 2) * C8 + kThreads - 1) / kThreads;
  vec_t reg[N][2];
  __device__ __forceinline__ void fetch(const T* __restrict__ base, int64_t stride, int row0, int row_end, int d, int tid) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + i * kThreads;
      const int row = row0 + 2 * (idx / C8), c8 = idx % C8;
      const bool ok = idx < (kChunk / 2) * C8 && c8 * 8 < d;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        if (ok && row + r < row_end) {
          reg[i][r] = *reinterpret_cast<const vec_t*>(base + (row + r) * stride + c8 * 8);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) reg[i][r][e] = static_cast<T>(0.f);
        }
      }
    }
  }
  __device__ __forceinline__ void commit(T* __restrict__ dst, int tid) const {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int idx = tid + i * kThreads;
      if (idx < (kChunk / 2) * C8) {
        const int r0 = 2 * (idx / C8), c8 = idx % C8;
        const int pos = (r0 & ~15) + vt_pos16(r0 & 15);  // even; row r0 + 1 lands at pos + 1
#pragma unroll
        for (int e = 0; e < 8; ++e)
          *reinterpret_cast<uint32_t*>(&dst[(c8 * 8 + e) * STR + pos]) = pack2<T>(reg[i][0][e], reg[i][1][e]);
      }
    }
  }
};

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

template <typename T, int DP>
__global__ __launch_bounds__(kThreads) void attn_bwd_dq_kernel(const AttnBwdParams p) {
  typedef typename Vec8<T>::type vec_t;
  constexpr int KSTEPS = DP / 16, MB = DP / 32;
  constexpr int RSTR = DP + 8, TSTR = kChunk + 8, OROW = DP * 2 + 16;
  constexpr int STAGE_BYTES = (2 * kChunk * RSTR + DP * TSTR) * 2;
  constexpr int TILE_BYTES = (kThreads / kWave) * 32 * OROW;
  __shared__ __attribute__((aligned(16))) uint8_t smem[STAGE_BYTES > TILE_BYTES ? STAGE_BYTES : TILE_BYTES];
  T* sK = reinterpret_cast<T*>(smem);   // [kChunk][RSTR]
  T* sV = sK + kChunk * RSTR;           // [kChunk][RSTR]
  T* sKt = sV + kChunk * RSTR;          // [DP][TSTR]

  const int blk = static_cast<int>(blockIdx.x % p.nblk);
  const int bh = static_cast<int>(blockIdx.x / p.nblk);
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

  RowStager<T, DP> k_rows, v_rows;
  TransStager<T, DP> k_cols;
  auto fetch = [&](int kc0) {
    k_rows.fetch(kb, p.ks[2], kc0, kv_end, p.d, tid);
    v_rows.fetch(vb, p.vs[2], kc0, kv_end, p.d, tid);
    k_cols.fetch(kb, p.ks[2], kc0, kv_end, p.d, tid);
  };
  if (kv_end > 0) fetch(0);
  for (int kc0 = 0; kc0 < kv_end; kc0 += kChunk) {
    if (kc0 > 0) __syncthreads();  // every wavefront is done reading the previous chunk
    k_rows.commit(sK, tid);
    v_rows.commit(sV, tid);
    k_cols.commit(sKt, tid);
    __syncthreads();
    if (kc0 + kChunk < kv_end) fetch(kc0 + kChunk);
#pragma unroll
    for (int kt = 0; kt < kChunk / 32; ++kt) {
      if (kc0 + kt * 32 >= kv_end || !wave_active) continue;  // wavefront-uniform
      if (p.causal && kc0 + kt * 32 > q_begin + wave * 32 + 31) continue;  // every key of the tile lies after the queries
      f32x16 sacc, dpacc;
#pragma unroll
      for (int j = 0; j < 16; ++j) sacc[j] = dpacc[j] = 0.f;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const vec_t ka = *reinterpret_cast<const vec_t*>(&sK[(kt * 32 + l32) * RSTR + 16 * s + 8 * hh]);
        const vec_t va = *reinterpret_cast<const vec_t*>(&sV[(kt * 32 + l32) * RSTR + 16 * s + 8 * hh]);
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
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float prob = __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -lse2));
        dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -delta_scaled));
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const vec_t a = *reinterpret_cast<const vec_t*>(&sKt[(mb * 32 + l32) * TSTR + kt * 32 + s2 * 16 + hh * 8]);
          dqacc[mb] = Mfma32<T>::run(a, dsb[s2], dqacc[mb]);
        }
    }
  }
  __syncthreads();  // the staging buffers now hold the output tiles
  store_owned<T, DP>(dqacc, smem + wave * (32 * OROW), dqb, p.dqs[2], q_begin + wave * 32, p.Tq, p.d, lane);
}

template <typename T, int DP>
__global__ __launch_bounds__(kThreads) void attn_bwd_dkv_kernel(const AttnBwdParams p) {
  typedef typename Vec8<T>::type vec_t;
  constexpr int KSTEPS = DP / 16, MB = DP / 32;
  constexpr int RSTR = DP + 8, TSTR = kChunk + 8, OROW = DP * 2 + 16;
  constexpr int STAGE_BYTES = (2 * kChunk * RSTR + 2 * DP * TSTR) * 2 + 2 * kChunk * 4;
  constexpr int TILE_BYTES = (kThreads / kWave) * 32 * OROW;
  __shared__ __attribute__((aligned(16))) uint8_t smem[STAGE_BYTES > TILE_BYTES ? STAGE_BYTES : TILE_BYTES];
  T* sQ = reinterpret_cast<T*>(smem);   // [kChunk][RSTR]
  T* sDo = sQ + kChunk * RSTR;          // [kChunk][RSTR]
  T* sQt = sDo + kChunk * RSTR;         // [DP][TSTR]
  T* sDot = sQt + DP * TSTR;            // [DP][TSTR]
  float* sLse = reinterpret_cast<float*>(sDot + DP * TSTR);  // [kChunk] base-2 log-sum-exp (+inf: row carries nothing)
  float* sDelta = sLse + kChunk;                             // [kChunk] D_i / sqrt(d)

  const int blk = static_cast<int>(blockIdx.x % p.nblk);
  const int bh = static_cast<int>(blockIdx.x / p.nblk);
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
    RowStager<T, DP> q_rows, do_rows;
    TransStager<T, DP> q_cols, do_cols;
    float lse_next = -INFINITY, delta_next = 0.f;
    auto fetch = [&](int qc0) {
      q_rows.fetch(qb, p.qs[2], qc0, q_valid, p.d, tid);
      do_rows.fetch(dob, p.dos[2], qc0, q_valid, p.d, tid);
      q_cols.fetch(qb, p.qs[2], qc0, q_valid, p.d, tid);
      do_cols.fetch(dob, p.dos[2], qc0, q_valid, p.d, tid);
      if (tid < kChunk) {
        const int qi = qc0 + tid;
        lse_next = qi < q_valid ? p.lse[stat0 + qi] : -INFINITY;
        delta_next = qi < q_valid ? p.delta[stat0 + qi] : 0.f;
      }
    };
    if (q_start < q_valid) fetch(q_start);
    for (int qc0 = q_start; qc0 < q_valid; qc0 += kChunk) {
      if (qc0 > q_start) __syncthreads();  // every wavefront is done reading the previous chunk
      q_rows.commit(sQ, tid);
      do_rows.commit(sDo, tid);
      q_cols.commit(sQt, tid);
      do_cols.commit(sDot, tid);
      if (tid < kChunk) {
        sLse[tid] = lse_next > -INFINITY ? lse_next * 1.4426950408889634f : INFINITY;  // exp2(x - inf) = 0
        sDelta[tid] = delta_next * p.scale;
      }
      __syncthreads();
      if (qc0 + kChunk < q_valid) fetch(qc0 + kChunk);
#pragma unroll
      for (int qt = 0; qt < kChunk / 32; ++qt) {
        if (qc0 + qt * 32 >= q_valid || k_begin + wave * 32 >= len) continue;  // wavefront-uniform
        if (p.causal && qc0 + qt * 32 + 31 < k_begin + wave * 32) continue;     // every query of the tile lies before the keys
        f32x16 sacc, dpacc;
#pragma unroll
        for (int j = 0; j < 16; ++j) sacc[j] = dpacc[j] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const vec_t qa = *reinterpret_cast<const vec_t*>(&sQ[(qt * 32 + l32) * RSTR + 16 * s + 8 * hh]);
          const vec_t da = *reinterpret_cast<const vec_t*>(&sDo[(qt * 32 + l32) * RSTR + 16 * s + 8 * hh]);
          sacc = Mfma32<T>::run(qa, kf[s], sacc);
          dpacc = Mfma32<T>::run(da, vf[s], dpacc);
        }
        // a padded key of the lane, or (causal) a query before the key: the score becomes -inf, the probability 0;
        // only a tile that crosses the causal diagonal needs per-element tests
        const bool diagonal = p.causal && qc0 + qt * 32 < k_begin + wave * 32 + 31;
        vec_t pb[2], dsb[2];
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          const int r0 = qt * 32 + jq * 8 + hh * 4;  // four consecutive queries of the chunk
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sLse[r0]);
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[r0]);  // already times 1 / sqrt(d)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = jq * 4 + e;
            float sc = k_ok ? sacc[j] : -INFINITY;
            if (diagonal && kj > qc0 + r0 + e) sc = -INFINITY;
            const float prob = __builtin_amdgcn_exp2f(fmaf(sc, c, -l4[e]));
            pb[j / 8][j % 8] = static_cast<T>(prob);
            dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -d4[e]));
          }
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const vec_t dot = *reinterpret_cast<const vec_t*>(&sDot[(mb * 32 + l32) * TSTR + qt * 32 + s2 * 16 + hh * 8]);
            const vec_t qt_ = *reinterpret_cast<const vec_t*>(&sQt[(mb * 32 + l32) * TSTR + qt * 32 + s2 * 16 + hh * 8]);
            dvacc[mb] = Mfma32<T>::run(dot, pb[s2], dvacc[mb]);
            dkacc[mb] = Mfma32<T>::run(qt_, dsb[s2], dkacc[mb]);
          }
      }
    }
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

template <typename T>
void launch_bwd(AttnBwdParams p, hipStream_t s) {
  p.nblk = static_cast<uint32_t>((p.Tq + kOwn - 1) / kOwn);
  p.total = p.nblk * p.B * p.H;
  if (p.d <= 32)
    hipLaunchKernelGGL((attn_bwd_dq_kernel<T, 32>), dim3(p.total), dim3(kThreads), 0, s, p);
  else
    hipLaunchKernelGGL((attn_bwd_dq_kernel<T, 64>), dim3(p.total), dim3(kThreads), 0, s, p);
  p.nblk = static_cast<uint32_t>((p.Tk + kOwn - 1) / kOwn);
  p.total = p.nblk * p.B * p.H;
  if (p.d <= 32)
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<T, 32>), dim3(p.total), dim3(kThreads), 0, s, p);
  else
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<T, 64>), dim3(p.total), dim3(kThreads), 0, s, p);
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
  using namespace taac;
  const char* name = "taac_flash_attn_bwd";
  if (B < 0 || H < 0 || Tq < 0 || Tk < 0 || d <= 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: negative dimension or non-positive head_dim", name);
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
  p.causal = is_causal ? 1 : 0;
  hipStream_t s = as_stream(stream);
  if (dtype == TAAC_BF16)
    launch_bwd<bf16_t>(p, s);
  else
    launch_bwd<f16_t>(p, s);
  return check_launch(name);
}
