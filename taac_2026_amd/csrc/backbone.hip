// Forward driver of the unified token backbone (pre-norm blocks + pCVR readout) and the readout kernel.
// The driver only sequences the library's own entry points on one stream over a caller-provided workspace.
#include <cstdlib>
#include <vector>

#include "common.h"

namespace taac {
namespace {

constexpr int kBlock = 256;

inline int64_t align256(int64_t v) { return (v + 255) & ~static_cast<int64_t>(255); }

// One workgroup per sample: fp32 sum over the valid prefix of the sample's tokens, mean, dot with the head weight,
// sigmoid. Thread layout: chunk = tid % (D/8) picks 8 features, group = tid / (D/8) strides over tokens.
__global__ __launch_bounds__(kBlock) void masked_mean_head_kernel(const bf16_t* __restrict__ x,
                                                                  const int32_t* __restrict__ lengths,
                                                                  const bf16_t* __restrict__ w_head,
                                                                  const bf16_t* __restrict__ b_head,
                                                                  float* __restrict__ p, int T, int D) {
  __shared__ float s_acc[kBlock][8];
  __shared__ float s_dot[kBlock];
  const int b = blockIdx.x;
  const int c8n = D / 8;
  const int groups = kBlock / c8n;
  const int chunk = threadIdx.x % c8n;
  const int group = threadIdx.x / c8n;
  int len = lengths[b];
  len = len < 0 ? 0 : (len > T ? T : len);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (group < groups) {
    const bf16_t* xb = x + static_cast<int64_t>(b) * T * D + chunk * 8;
    for (int t = group; t < len; t += groups) {
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(xb + static_cast<int64_t>(t) * D);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += static_cast<float>(v[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) s_acc[threadIdx.x][e] = acc[e];
  __syncthreads();
  float dot = 0.f;
  if (threadIdx.x < c8n) {
    const float denom = static_cast<float>(len < 1 ? 1 : len);
    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(w_head + threadIdx.x * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float s = 0.f;
      for (int g = 0; g < groups; ++g) s += s_acc[g * c8n + threadIdx.x][e];
      dot += (s / denom) * static_cast<float>(wv[e]);
    }
  }
  s_dot[threadIdx.x] = dot;
  __syncthreads();
  if (threadIdx.x == 0) {
    float z = b_head != nullptr ? static_cast<float>(b_head[0]) : 0.f;
    for (int i = 0; i < c8n; ++i) z += s_dot[i];
    p[b] = 1.0f / (1.0f + expf(-z));
  }
}

// The same readout from per-token dot products with the head weight (left behind by the last block's kernel): one
// wavefront per sample adds the dots of its valid prefix in a fixed order, mean, bias, sigmoid.
__global__ __launch_bounds__(kBlock) void token_dots_head_kernel(const float* __restrict__ dots,
                                                                 const int32_t* __restrict__ lengths,
                                                                 const bf16_t* __restrict__ b_head, float* __restrict__ p,
                                                                 int B, int T) {
  const int b = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  if (b >= B) return;
  int len = lengths[b];
  len = len < 0 ? 0 : (len > T ? T : len);
  const float* row = dots + static_cast<int64_t>(b) * T;
  float s = 0.f;
  for (int t = lane; t < len; t += kWave) s += row[t];
  s = group_sum<kWave>(s);
  if (lane == 0) {
    const float z = (b_head != nullptr ? static_cast<float>(b_head[0]) : 0.f) + s / static_cast<float>(len < 1 ? 1 : len);
    p[b] = 1.0f / (1.0f + expf(-z));
  }
}

// Number of valid tokens of sample b: its clamped length, or the set bits among the first T of its bit row.
__device__ __forceinline__ int32_t valid_count(const int32_t* __restrict__ lengths, const uint32_t* __restrict__ bits,
                                               int b, int T) {
  if (lengths != nullptr) {
    const int32_t len = lengths[b];
    return len < 0 ? 0 : (len > T ? T : len);
  }
  const int wpr = (T + 31) / 32;
  int32_t n = 0;
  for (int w = 0; w < wpr; ++w) {
    uint32_t word = bits[static_cast<int64_t>(b) * wpr + w];
    if (w == wpr - 1 && T % 32 != 0) word &= (1u << (T % 32)) - 1u;
    n += __popc(word);
  }
  return n;
}

// Exclusive prefix sums of the per-sample valid counts (one workgroup; B is walked in slabs of kBlock with a running
// carry).
__global__ __launch_bounds__(kBlock) void length_offsets_kernel(const int32_t* __restrict__ lengths,
                                                                const uint32_t* __restrict__ bits, int B, int T,
                                                                int32_t* __restrict__ offsets,
                                                                int32_t* __restrict__ n_rows) {
  __shared__ int32_t s_scan[kBlock];
  int32_t carry = 0;
  for (int base = 0; base < B; base += kBlock) {
    const int b = base + threadIdx.x;
    const int32_t len = b < B ? valid_count(lengths, bits, b, T) : 0;
    s_scan[threadIdx.x] = len;
    __syncthreads();
    for (int step = 1; step < kBlock; step <<= 1) {  // inclusive scan, Hillis-Steele
      const int32_t add = threadIdx.x >= step ? s_scan[threadIdx.x - step] : 0;
      __syncthreads();
      s_scan[threadIdx.x] += add;
      __syncthreads();
    }
    if (b < B) offsets[b] = carry + s_scan[threadIdx.x] - len;
    carry += s_scan[kBlock - 1];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    offsets[B] = carry;
    *n_rows = carry;
  }
}

__global__ __launch_bounds__(kBlock) void valid_rows_kernel(const int32_t* __restrict__ lengths,
                                                            const int32_t* __restrict__ offsets, int T,
                                                            int32_t* __restrict__ rows) {
  const int b = blockIdx.y;
  int32_t len = lengths[b];
  len = len < 0 ? 0 : (len > T ? T : len);
  const int t = blockIdx.x * kBlock + threadIdx.x;
  if (t < len) rows[offsets[b] + t] = b * T + t;
}

// The same for a validity bit row per sample: token t goes to slot offsets[b] + (number of valid tokens before t).
__global__ __launch_bounds__(kBlock) void valid_rows_bits_kernel(const uint32_t* __restrict__ bits,
                                                                 const int32_t* __restrict__ offsets, int T,
                                                                 int32_t* __restrict__ rows) {
  const int b = blockIdx.y;
  const int t = blockIdx.x * kBlock + threadIdx.x;
  if (t >= T) return;
  const int wpr = (T + 31) / 32;
  const uint32_t* row = bits + static_cast<int64_t>(b) * wpr;
  const uint32_t word = row[t / 32];
  if (((word >> (t % 32)) & 1u) == 0u) return;
  int32_t rank = __popc(word & ((1u << (t % 32)) - 1u));
  for (int w = 0; w < t / 32; ++w) rank += __popc(row[w]);
  rows[offsets[b] + rank] = b * T + t;
}

// front_rows[i] = b * T + (i - offsets[b]) for token i of sample b = rows[i] / T; lengths[b] = offsets[b + 1] - offsets[b].
__global__ __launch_bounds__(kBlock) void front_rows_kernel(const int32_t* __restrict__ rows,
                                                            const int32_t* __restrict__ n_rows, int B, int T,
                                                            int32_t* __restrict__ front_rows,
                                                            int32_t* __restrict__ lengths) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int32_t* offsets = rows + static_cast<int64_t>(B) * T;
  if (i < B) lengths[i] = offsets[i + 1] - offsets[i];
  if (i >= *n_rows) return;
  const int b = rows[i] / T;
  front_rows[i] = b * T + static_cast<int32_t>(i - offsets[b]);
}

// One workgroup per (sample b, 32 front rows): the sample's key positions go to LDS once; a wavefront then takes 8
// rows, holds a row's structure words across its lanes (lane l: words l and l + 64) and, 64 keys per step, lets lane j
// pick the word of its key from them with a lane permute; a ballot gathers the bits. Only rows below the sample's
// number of valid tokens n_b are written, and of those the words that hold a key below n_b (the attention kernel reads
// nothing else), bits at or beyond n_b as zeros.
constexpr int kFrontRowsPerBlock = 32;
__global__ __launch_bounds__(kBlock) void mask_front_bits_kernel(const uint32_t* __restrict__ struct_bits, int T,
                                                                 const int32_t* __restrict__ rows, int B,
                                                                 uint32_t* __restrict__ out) {
  __shared__ uint16_t kpos[4096];
  const int wpr = (T + 31) / 32;
  const int slabs = (T + kFrontRowsPerBlock - 1) / kFrontRowsPerBlock;
  const int b = blockIdx.x / slabs, r0 = (blockIdx.x % slabs) * kFrontRowsPerBlock;
  const int32_t* offsets = rows + static_cast<int64_t>(B) * T;
  const int32_t off = offsets[b];
  const int n = offsets[b + 1] - off;
  if (r0 >= n) return;  // workgroup-uniform
  for (int j = threadIdx.x; j < n; j += kBlock) kpos[j] = static_cast<uint16_t>(rows[off + j] - b * T);
  __syncthreads();
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  constexpr int kRowsPerWave = kFrontRowsPerBlock / (kBlock / kWave);
  // the structure words of the wavefront's rows first (independent loads), then the gathers
  uint32_t w_lo[kRowsPerWave], w_hi[kRowsPerWave];
#pragma unroll
  for (int i = 0; i < kRowsPerWave; ++i) {
    const int r = r0 + wave * kRowsPerWave + i;
    const uint32_t* src = struct_bits + static_cast<int64_t>(kpos[r < n ? r : 0]) * wpr;
    w_lo[i] = (r < n && lane < wpr) ? src[lane] : 0u;
    w_hi[i] = (r < n && lane + kWave < wpr) ? src[lane + kWave] : 0u;
  }
  for (int j0 = 0; j0 < n; j0 += kWave) {
    const int j = j0 + lane;
    const int key = j < n ? kpos[j] : 0;
    const int src_lane = (key >> 5) & (kWave - 1);
    const bool upper = (key >> 5) >= kWave;
#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) {
      const int r = r0 + wave * kRowsPerWave + i;
      if (r >= n) break;  // wavefront-uniform
      const uint32_t lo = __shfl(w_lo[i], src_lane, kWave);
      const uint32_t word = wpr > kWave ? (upper ? __shfl(w_hi[i], src_lane, kWave) : lo) : lo;
      const uint64_t bits = __builtin_amdgcn_ballot_w64(j < n && ((word >> (key & 31)) & 1u) != 0u);
      uint32_t* dst = out + (static_cast<int64_t>(b) * T + r) * wpr;
      if (lane < 2 && j0 / 32 + lane < wpr) dst[j0 / 32 + lane] = static_cast<uint32_t>(bits >> (32 * lane));
    }
  }
}

// prod[d] = wq[d] * wk[d] in fp32: the weights of a query and a key norm act on an attention score only through their
// product, which the attention kernel applies to the query features.
__global__ __launch_bounds__(kBlock) void weight_product_kernel(const bf16_t* __restrict__ wq,
                                                                const bf16_t* __restrict__ wk,
                                                                float* __restrict__ prod, int D) {
  const int d = blockIdx.x * kBlock + threadIdx.x;
  if (d < D) prod[d] = static_cast<float>(wq[d]) * static_cast<float>(wk[d]);
}

// Zero-fills the rows of the padded positions of x [B, T, D] (16 bytes per thread).
__global__ __launch_bounds__(kBlock) void zero_padded_rows_kernel(bf16_t* __restrict__ x,
                                                                  const int32_t* __restrict__ lengths, int T, int D) {
  const int b = blockIdx.y;
  int32_t len = lengths[b];
  len = len < 0 ? 0 : (len > T ? T : len);
  const int c8n = D / 8;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t t = len + idx / c8n;
  if (t >= T) return;
  bf16x8 z;
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = static_cast<bf16_t>(0.f);
  *reinterpret_cast<bf16x8*>(x + (static_cast<int64_t>(b) * T + t) * D + (idx % c8n) * 8) = z;
}

}  // namespace
}  // namespace taac

namespace taac {
namespace {
// One 16-byte piece per thread: row (b, t) of out is a[offsets[b] + t] (+ b2 of the same row) when t < lengths[b], else
// the row of `padded`.
__global__ __launch_bounds__(kBlock) void rows_merge_kernel(const bf16x8* __restrict__ padded, const bf16x8* __restrict__ a,
                                                            const bf16x8* __restrict__ b2,
                                                            const int32_t* __restrict__ lengths,
                                                            const int32_t* __restrict__ offsets, bf16x8* __restrict__ out,
                                                            int64_t pieces_total, int T, int pieces) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= pieces_total) return;
  const int64_t row = idx / pieces;
  const int c = static_cast<int>(idx % pieces);
  const int b = static_cast<int>(row / T), t = static_cast<int>(row % T);
  int32_t len = lengths[b];
  len = len < 0 ? 0 : (len > T ? T : len);
  bf16x8 v;
  if (t < len) {
    const int64_t src = (static_cast<int64_t>(offsets[b]) + t) * pieces + c;
    v = a[src];
    if (b2 != nullptr) {
      const bf16x8 w = b2[src];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) + static_cast<float>(w[e]));
    }
  } else {
    v = padded[idx];
  }
  out[idx] = v;
}

// The same merge for padding that is not a prefix: (b, t) is valid iff bit t of valid_bits[b] is set, and its compact row
// is offsets[b] + the number of valid tokens of the sample in front of it (word_prefix[b][w], if given, = the number of
// valid tokens in the words before word w, which saves the walk over those words).
__global__ __launch_bounds__(kBlock) void rows_merge_bits_kernel(const bf16x8* __restrict__ padded,
                                                                 const bf16x8* __restrict__ a, const bf16x8* __restrict__ b2,
                                                                 const uint32_t* __restrict__ valid_bits,
                                                                 const int32_t* __restrict__ word_prefix,
                                                                 const int32_t* __restrict__ offsets, bf16x8* __restrict__ out,
                                                                 int64_t pieces_total, int T, int pieces) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= pieces_total) return;
  const int64_t row = idx / pieces;
  const int c = static_cast<int>(idx % pieces);
  const int b = static_cast<int>(row / T), t = static_cast<int>(row % T);
  const uint32_t* bits = valid_bits + static_cast<int64_t>(b) * ((T + 31) / 32);
  const uint32_t word = bits[t / 32];
  bf16x8 v;
  if ((word >> (t % 32)) & 1u) {
    int rank = __popc(word & ((1u << (t % 32)) - 1u));
    if (word_prefix != nullptr) {
      rank += word_prefix[static_cast<int64_t>(b) * ((T + 31) / 32) + t / 32];
    } else {
      for (int w = 0; w < t / 32; ++w) rank += __popc(bits[w]);
    }
    const int64_t src = (static_cast<int64_t>(offsets[b]) + rank) * pieces + c;
    v = a[src];
    if (b2 != nullptr) {
      const bf16x8 w2 = b2[src];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) + static_cast<float>(w2[e]));
    }
  } else {
    v = padded[idx];
  }
  out[idx] = v;
}

// dst[i] = src[rows[i]] for i < n: one 16-byte piece per thread.
__global__ __launch_bounds__(kBlock) void rows_gather_kernel(const bf16x8* __restrict__ src, int64_t src_pieces,
                                                             const int32_t* __restrict__ rows, bf16x8* __restrict__ dst,
                                                             int64_t pieces_total, int pieces) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= pieces_total) return;
  const int64_t i = idx / pieces;
  const int c = static_cast<int>(idx % pieces);
  dst[idx] = __builtin_nontemporal_load(src + static_cast<int64_t>(rows[i]) * src_pieces + c);
}
}  // namespace
}  // namespace taac

extern "C" int taac_rows_gather(const void* src, int64_t ld_src, const int32_t* rows, int64_t n, void* dst, int32_t W,
                                void* stream) {
  using namespace taac;
  const char* name = "taac_rows_gather";
  if (n < 0 || W <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (W % 8 != 0 || ld_src % 8 != 0 || ld_src < W)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: W and the source row stride must be multiples of 8 and cover a row", name);
  if (n == 0) return TAAC_OK;
  if (!src || !rows || !dst) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!aligned16(src) || !aligned16(dst)) return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int64_t pieces_total = n * (W / 8);
  const int64_t blocks = (pieces_total + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(rows_gather_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const bf16x8*>(src), ld_src / 8, rows, static_cast<bf16x8*>(dst), pieces_total, W / 8);
  return check_launch(name);
}

extern "C" int taac_rows_merge(const void* padded, const void* compact_a, const void* compact_b, const int32_t* key_lengths,
                               const int32_t* offsets, void* out, int32_t B, int32_t T, int32_t W, void* stream) {
  using namespace taac;
  const char* name = "taac_rows_merge";
  if (B < 0 || T < 0 || W <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (W % 8 != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: W=%d must be a multiple of 8", name, W);
  if (B == 0 || T == 0) return TAAC_OK;
  if (!padded || !compact_a || !key_lengths || !offsets || !out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!aligned16(padded) || !aligned16(compact_a) || !aligned16(compact_b) || !aligned16(out))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int64_t pieces_total = static_cast<int64_t>(B) * T * (W / 8);
  const int64_t blocks = (pieces_total + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(rows_merge_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const bf16x8*>(padded), static_cast<const bf16x8*>(compact_a),
                     static_cast<const bf16x8*>(compact_b), key_lengths, offsets, static_cast<bf16x8*>(out), pieces_total, T,
                     W / 8);
  return check_launch(name);
}

extern "C" int taac_rows_merge_bits(const void* padded, const void* compact_a, const void* compact_b,
                                    const uint32_t* valid_bits, const int32_t* word_prefix, const int32_t* offsets,
                                    void* out, int32_t B, int32_t T, int32_t W, void* stream) {
  using namespace taac;
  const char* name = "taac_rows_merge_bits";
  if (B < 0 || T < 0 || W <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (W % 8 != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: W=%d must be a multiple of 8", name, W);
  if (B == 0 || T == 0) return TAAC_OK;
  if (!padded || !compact_a || !valid_bits || !offsets || !out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!aligned16(padded) || !aligned16(compact_a) || !aligned16(compact_b) || !aligned16(out))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int64_t pieces_total = static_cast<int64_t>(B) * T * (W / 8);
  const int64_t blocks = (pieces_total + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(rows_merge_bits_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const bf16x8*>(padded), static_cast<const bf16x8*>(compact_a),
                     static_cast<const bf16x8*>(compact_b), valid_bits, word_prefix, offsets, static_cast<bf16x8*>(out),
                     pieces_total, T, W / 8);
  return check_launch(name);
}

extern "C" int taac_valid_rows(const int32_t* key_lengths, int32_t B, int32_t T, int32_t* rows, int32_t* n_rows,
                               void* stream) {
  using namespace taac;
  const char* name = "taac_valid_rows";
  if (B < 0 || T < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (static_cast<int64_t>(B) * T > 0x7fffffffLL - B - 1)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: B * T must fit 32-bit row numbers", name);
  if (!rows || !n_rows || (B > 0 && !key_lengths)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (B > 65535) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 65535 samples", name);
  int32_t* offsets = rows + static_cast<int64_t>(B) * T;
  hipLaunchKernelGGL(length_offsets_kernel, dim3(1), dim3(kBlock), 0, as_stream(stream), key_lengths,
                     static_cast<const uint32_t*>(nullptr), B, T, offsets, n_rows);
  if (B > 0 && T > 0)
    hipLaunchKernelGGL(valid_rows_kernel, dim3((T + kBlock - 1) / kBlock, B), dim3(kBlock), 0, as_stream(stream),
                       key_lengths, offsets, T, rows);
  return check_launch(name);
}

extern "C" int taac_valid_rows_from_bits(const uint32_t* valid_bits, int32_t B, int32_t T, int32_t* rows,
                                         int32_t* n_rows, void* stream) {
  using namespace taac;
  const char* name = "taac_valid_rows_from_bits";
  if (B < 0 || T < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (static_cast<int64_t>(B) * T > 0x7fffffffLL - B - 1)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: B * T must fit 32-bit row numbers", name);
  if (!rows || !n_rows || (B > 0 && T > 0 && !valid_bits)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (B > 65535) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 65535 samples", name);
  int32_t* offsets = rows + static_cast<int64_t>(B) * T;
  hipLaunchKernelGGL(length_offsets_kernel, dim3(1), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const int32_t*>(nullptr), valid_bits, B, T, offsets, n_rows);
  if (B > 0 && T > 0)
    hipLaunchKernelGGL(valid_rows_bits_kernel, dim3((T + kBlock - 1) / kBlock, B), dim3(kBlock), 0, as_stream(stream),
                       valid_bits, offsets, T, rows);
  return check_launch(name);
}

extern "C" int taac_masked_mean_head(const void* x, const int32_t* lengths, const void* w_head, const void* b_head,
                                     float* p, int32_t B, int32_t T, int32_t D, void* stream) {
  using namespace taac;
  const char* name = "taac_masked_mean_head";
  if (B < 0 || T < 0 || D <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (D % 8 != 0 || D > 8 * kBlock)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D=%d must be a multiple of 8 and at most %d", name, D, 8 * kBlock);
  if (B == 0) return TAAC_OK;
  if (!x || !lengths || !w_head || !p) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!aligned16(x) || !aligned16(w_head))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: x and w_head must be 16-byte aligned", name);
  hipLaunchKernelGGL(masked_mean_head_kernel, dim3(B), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const bf16_t*>(x), lengths, static_cast<const bf16_t*>(w_head),
                     static_cast<const bf16_t*>(b_head), p, T, D);
  return check_launch(name);
}

namespace taac {
namespace {
// Fused (token-stationary) path: model widths 128 / 256, hidden size a multiple of 32.
inline bool fused_shape(int32_t D, int32_t F) { return (D == 128 || D == 256) && F % 32 == 0; }
// Fragment-ordered weights of one block: qkv, out, feed-forward.
// Row index of the valid tokens: B*T rows + B+1 offsets + the count.
inline int64_t row_index_bytes(int32_t B, int32_t T) { return align256((static_cast<int64_t>(B) * T + B + 2) * 4); }
inline int64_t packed_block_bytes(int32_t D, int32_t F) {
  return align256(static_cast<int64_t>(3) * D * D * 2) + align256(static_cast<int64_t>(D) * D * 2) +
         align256(static_cast<int64_t>(3) * D * F * 2);
}
// Query / key norm scratch of the fused path: per-chunk sums of squares [2D / 64, M], factors [2, M], the
// concatenated query | key norm weights [2D].
inline int64_t qk_norm_bytes(int64_t M, int32_t D) {
  return align256((2 * D / 64) * M * 4) + align256(2 * M * 4) + align256(static_cast<int64_t>(D) * 4);
}
// FP8 mode (TAAC_BACKBONE_FP8; D = 256, F a multiple of 64): per block the e4m3 qkv / out weights, the packed feed-forward
// blob and 8 scales (weights: qkv, out, up, down; activations: block input, attention output, feed-forward input, gated
// hidden state); one more set of scales behind the last block.
inline bool fp8_shape(int32_t D, int32_t F) { return D == 256 && F % 64 == 0; }
inline int64_t fp8_block_bytes(int32_t D, int32_t F) {
  return align256(static_cast<int64_t>(3) * D * D) + align256(static_cast<int64_t>(D) * D) +
         align256(taac_ffn_fp8_packed_bytes(D, F));
}
inline int64_t fp8_bytes(int32_t D, int32_t F, int32_t n_blocks) {
  return fp8_shape(D, F) ? n_blocks * fp8_block_bytes(D, F) + align256((n_blocks + 1) * 8 * 4) : 0;
}
}  // namespace
}  // namespace taac

extern "C" int64_t taac_backbone_workspace_bytes(int32_t B, int32_t T, int32_t D, int32_t F, int32_t n_blocks) {
  using namespace taac;
  if (B < 0 || T < 0 || D <= 0 || F <= 0 || n_blocks < 0) return -1;
  const int64_t M = static_cast<int64_t>(B) * T;
  // x, h (shared with the attention output), qkv, then either the packed weights + the valid-row index (fused path)
  // or the gated hidden state
  const int64_t acts = align256(M * D * 2) * 2 + align256(M * 3 * D * 2);
  return acts + (fused_shape(D, F) ? n_blocks * packed_block_bytes(D, F) + row_index_bytes(B, T) + qk_norm_bytes(M, D) +
                                         fp8_bytes(D, F, n_blocks)
                                   : align256(M * F * 2));
}

extern "C" int64_t taac_backbone_fp8_scales_offset(int32_t B, int32_t T, int32_t D, int32_t F, int32_t n_blocks) {
  using namespace taac;
  if (B < 0 || T < 0 || n_blocks < 0 || !fp8_shape(D, F)) return -1;
  return taac_backbone_workspace_bytes(B, T, D, F, n_blocks) - align256((n_blocks + 1) * 8 * 4);
}

extern "C" int taac_backbone_fwd(const void* emb, const int32_t* key_lengths, const taac_block_weights* blocks,
                                 int32_t n_blocks, const void* w_head, const void* b_head, int32_t B, int32_t T,
                                 int32_t D, int32_t heads, int32_t F, float eps, const void* rope_cos_sin,
                                 int flags, void* workspace, int64_t workspace_bytes, void* hidden_out, float* p,
                                 void* stream) {
  using namespace taac;
  const char* name = "taac_backbone_fwd";
  if (flags & ~(TAAC_BACKBONE_DENSE_TOKENS | TAAC_BACKBONE_SPLIT_OUT_FFN | TAAC_BACKBONE_FP8 | TAAC_BACKBONE_ROW_MAJOR_QKV))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown flag bits (%d)", name, flags);
  const bool fp8 = (flags & TAAC_BACKBONE_FP8) != 0;
  if (fp8 && !fp8_shape(D, F))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: the FP8 dense layers are built for D = 256 and F a multiple of 64", name);
  if (fp8 && rope_cos_sin != nullptr)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: the FP8 mode covers the plain attention layer (no rotary embedding)", name);
  if (B < 0 || T < 0 || D <= 0 || F <= 0 || heads <= 0 || n_blocks < 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (D % heads != 0 || (D / heads) % 8 != 0 || D / heads > 128)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D=%d heads=%d: head_dim must be a multiple of 8, at most 128", name, D,
                     heads);
  if (D % 8 != 0 || F % 8 != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: D and F must be multiples of 8", name);
  if (B == 0 || T == 0) return TAAC_OK;
  if (!emb || !key_lengths || !p || !w_head || (n_blocks > 0 && !blocks))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int64_t need = taac_backbone_workspace_bytes(B, T, D, F, n_blocks);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: workspace must be 256-byte aligned and hold %lld bytes", name,
                     (long long)need);

  const int64_t M = static_cast<int64_t>(B) * T;
  char* ws = static_cast<char*>(workspace);
  bf16_t* x = reinterpret_cast<bf16_t*>(ws);
  ws += align256(M * D * 2);
  bf16_t* h = reinterpret_cast<bf16_t*>(ws);
  ws += align256(M * D * 2);
  bf16_t* qkv = reinterpret_cast<bf16_t*>(ws);
  ws += align256(M * 3 * D * 2);
  bf16_t* g = reinterpret_cast<bf16_t*>(ws);  // unfused path: gated hidden state; fused path: packed weights
  char* packed = ws;
  const bool fused = fused_shape(D, F);
  // the packed up projection carries the constants of the gate's activation where the kernels take them from there
  const bool fold_act = fused && ffn_act_fold_supported(D, F);
  // Fused path: the dense layers walk the valid tokens only (row index built from key_lengths on the device); the
  // padded positions of the residual stream are never read or written. TAAC_BACKBONE_DENSE_TOKENS switches this off.
  int32_t* rows = nullptr;
  int32_t* n_rows = nullptr;
  char* after_packed = packed + static_cast<int64_t>(n_blocks) * packed_block_bytes(D, F);
  float* qk_sumsq = reinterpret_cast<float*>(after_packed + row_index_bytes(B, T));
  float* qk_rstd = reinterpret_cast<float*>(reinterpret_cast<char*>(qk_sumsq) + align256((2 * D / 64) * M * 4));
  bf16_t* qk_weight = reinterpret_cast<bf16_t*>(reinterpret_cast<char*>(qk_rstd) + align256(2 * M * 4));
  if (rope_cos_sin != nullptr && !aligned16(rope_cos_sin))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: the rotary table must be 16-byte aligned", name);
  if (fused && n_blocks > 0 && !(flags & TAAC_BACKBONE_DENSE_TOKENS)) {
    rows = reinterpret_cast<int32_t*>(after_packed);
    n_rows = rows + M + B + 1;
    const int rc_rows = taac_valid_rows(key_lengths, B, T, rows, n_rows, stream);
    if (rc_rows != TAAC_OK) return rc_rows;
  }

  const int dh = D / heads;
  const int64_t qkv_strides[4] = {static_cast<int64_t>(T) * 3 * D, dh, 3 * static_cast<int64_t>(D), 1};
  const int64_t o_strides[4] = {static_cast<int64_t>(T) * D, dh, D, 1};

  const bf16_t* cur = static_cast<const bf16_t*>(emb);
  int rc;
  // TAAC_BACKBONE_SPLIT_OUT_FFN: the out projection and the feed-forward half as two kernels (comparison route).
  const bool split_out_ffn = (flags & TAAC_BACKBONE_SPLIT_OUT_FFN) != 0;
  if (fused && !fp8 && n_blocks > 0) {
    // One launch re-lays the weights of all blocks into fragment order.
    std::vector<void*> pk(3 * static_cast<size_t>(n_blocks));
    for (int i = 0; i < n_blocks; ++i) {
      const taac_block_weights& w = blocks[i];
      if (!w.qkv_weight || !w.out_weight || !w.up_weight || !w.down_weight)
        return set_error(TAAC_ERR_INVALID_VALUE, "%s: block %d has a null weight", name, i);
      char* base = packed + static_cast<int64_t>(i) * packed_block_bytes(D, F);
      pk[i] = base;
      pk[n_blocks + i] = base + align256(static_cast<int64_t>(3) * D * D * 2);
      pk[2 * n_blocks + i] = base + align256(static_cast<int64_t>(3) * D * D * 2) + align256(static_cast<int64_t>(D) * D * 2);
    }
    if ((rc = pack_backbone_blocks(blocks, n_blocks, D, F, pk.data(), pk.data() + n_blocks, pk.data() + 2 * n_blocks,
                                   fold_act, as_stream(stream), name)) != TAAC_OK)
      return rc;
  }
  // FP8 mode: scales and e4m3 weights of all blocks (three launches), then the scale of the first block's input
  char* fp8_base = reinterpret_cast<char*>(qk_weight) + align256(static_cast<int64_t>(D) * 4);
  float* fp8_scales = reinterpret_cast<float*>(fp8_base + static_cast<int64_t>(n_blocks) * (fp8 ? fp8_block_bytes(D, F) : 0));
  auto fp8_qkv = [&](int i) { return fp8_base + static_cast<int64_t>(i) * fp8_block_bytes(D, F); };
  auto fp8_out = [&](int i) { return fp8_qkv(i) + align256(static_cast<int64_t>(3) * D * D); };
  auto fp8_ffn = [&](int i) { return fp8_out(i) + align256(static_cast<int64_t>(D) * D); };
  if (fp8 && n_blocks > 0) {
    std::vector<float*> sc(n_blocks);
    std::vector<void*> wq(3 * static_cast<size_t>(n_blocks));
    for (int i = 0; i < n_blocks; ++i) {
      if (blocks[i].query_norm_weight || blocks[i].key_norm_weight)
        return set_error(TAAC_ERR_UNSUPPORTED, "%s: the FP8 mode covers the plain attention layer (no query / key norm)", name);
      if (!blocks[i].attn_norm_weight || !blocks[i].ffn_norm_weight)
        return set_error(TAAC_ERR_INVALID_VALUE, "%s: block %d has a null weight", name, i);
      sc[i] = fp8_scales + 8 * i;
      wq[i] = fp8_qkv(i);
      wq[n_blocks + i] = fp8_out(i);
      wq[2 * n_blocks + i] = fp8_ffn(i);
    }
    if ((rc = fill_zero(fp8_scales, (n_blocks + 1) * 8, as_stream(stream), name)) != TAAC_OK) return rc;
    if ((rc = prepare_backbone_fp8(blocks, n_blocks, D, F, sc.data(), wq.data(), wq.data() + n_blocks,
                                   wq.data() + 2 * n_blocks, as_stream(stream), name)) != TAAC_OK)
      return rc;
    if ((rc = rmsnorm_amax_256(emb, D, blocks[0].attn_norm_weight, eps, M, rows, n_rows, fp8_scales + 4, as_stream(stream),
                               name)) != TAAC_OK)
      return rc;
  }
  // Plain attention layers (no query / key norm, no rotary embedding) with heads of 32 or 64 features keep q | k | v and
  // the attention output as stacks of per-head planes [3 * heads][M][dh] / [heads][M][dh] instead of [M][3 * D] / [M][D]
  // rows: a head's rows are then contiguous for the attention kernel (64-byte pieces of 1 536-byte rows otherwise), and the
  // dense kernels on either side address the planes directly. TAAC_BACKBONE_ROW_MAJOR_QKV keeps the rows (same results).
  const bool planes = fused && !fp8 && !split_out_ffn && (dh == 32 || dh == 64) && !(flags & TAAC_BACKBONE_ROW_MAJOR_QKV);
  const int64_t plane_elems = M * dh;
  const int64_t plane_strides[4] = {static_cast<int64_t>(T) * dh, plane_elems, dh, 1};
  // The last block's kernel (out projection + feed-forward in one) also leaves every token's dot product with the head
  // weight behind, in the q | k | v buffer that is free by then: the readout adds M floats instead of reading the final
  // hidden state again.
  float* token_dots = reinterpret_cast<float*>(qkv);
  const bool head_rides = aligned16(w_head);
  bool dots_ready = false;
  for (int i = 0; i < n_blocks; ++i) {
    const taac_block_weights& w = blocks[i];
    if (!w.attn_norm_weight || !w.qkv_weight || !w.out_weight || !w.ffn_norm_weight || !w.up_weight || !w.down_weight)
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: block %d has a null weight", name, i);
    const bool last = (i == n_blocks - 1);
    const bool ride = last && head_rides;
    bf16_t* x_out = (last && hidden_out != nullptr) ? static_cast<bf16_t*>(hidden_out) : x;
    if (fp8) {
      // Four dense layers with e4m3 operands and per-tensor scales; every activation scale comes out of the epilogue of the
      // kernel that produces the tensor (scales[4..7] = block input, attention output, feed-forward input, hidden state).
      float* sc = fp8_scales + 8 * i;
      PreclearedMaxima precleared;
      if ((rc = taac_norm_linear_fp8_fwd(cur, D, w.attn_norm_weight, eps, fp8_qkv(i), w.qkv_bias, sc + 4, sc + 0, nullptr, 0,
                                         qkv, 3 * D, M, 3 * D, D, rows, n_rows, nullptr, 0.f, nullptr, stream)) != TAAC_OK)
        return rc;
      if ((rc = taac_flash_attn_amax_fwd(qkv, qkv + D, qkv + 2 * D, key_lengths, nullptr, nullptr, nullptr, h, sc + 5, B,
                                         heads, T, T, D / heads, qkv_strides, qkv_strides, qkv_strides, o_strides, 0,
                                         rows ? 2 : 1, TAAC_BF16, stream)) != TAAC_OK)
        return rc;
      if ((rc = taac_norm_linear_fp8_fwd(h, D, nullptr, eps, fp8_out(i), w.out_bias, sc + 5, sc + 1, cur, D, x, D, M, D, D,
                                         rows, n_rows, w.ffn_norm_weight, eps, sc + 6, stream)) != TAAC_OK)
        return rc;
      if ((rc = taac_swiglu_ffn_fp8_fwd(x, D, w.ffn_norm_weight, eps, fp8_ffn(i), w.up_bias, w.down_bias, sc + 6, sc + 2,
                                        sc + 3, sc + 7, x, D, x_out, D, M, D, F, 1, rows, n_rows,
                                        last ? nullptr : blocks[i + 1].attn_norm_weight, eps, last ? nullptr : sc + 8 + 4,
                                        stream)) != TAAC_OK)
        return rc;
      cur = x_out;
      continue;
    }
    // Fused path: token-stationary kernels with norms and residuals fused, weights repacked into fragment order.
    char* pk_qkv = packed + static_cast<int64_t>(i) * packed_block_bytes(D, F);
    char* pk_out = pk_qkv + align256(static_cast<int64_t>(3) * D * D * 2);
    char* pk_ffn = pk_out + align256(static_cast<int64_t>(D) * D * 2);
    const int ffn_folded = (w.ffn_norm_weight != nullptr ? TAAC_FOLDED_NORM : 0) | (fold_act ? TAAC_FOLDED_ACTIVATION : 0);
    // attention half
    if ((w.query_norm_weight == nullptr) != (w.key_norm_weight == nullptr))
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: block %d: query and key norm weights come together", name, i);
    const bool qk_norm = w.query_norm_weight != nullptr;
    const bool qk_prepare = qk_norm || rope_cos_sin != nullptr;
    const float* q_scale = nullptr;
    const float* k_scale = nullptr;
    const float* q_col_scale = nullptr;
    if (fused && qk_prepare) {
      // The norm statistic comes out of the projection's epilogue and the per-token factor of the norm is applied by
      // the attention kernel. Without a rotation the two norm weights go to the attention kernel as well, as their
      // product on the query features; with one, the epilogue applies weight and rotation. Either way there is no
      // pass of its own over q and k.
      const bool weights_in_epilogue = qk_norm && rope_cos_sin != nullptr;
      if (qk_norm && !weights_in_epilogue) {
        float* prod = reinterpret_cast<float*>(qk_weight);
        hipLaunchKernelGGL(weight_product_kernel, dim3((D + kBlock - 1) / kBlock), dim3(kBlock), 0, as_stream(stream),
                           static_cast<const bf16_t*>(w.query_norm_weight),
                           static_cast<const bf16_t*>(w.key_norm_weight), prod, D);
        if ((rc = check_launch(name)) != TAAC_OK) return rc;
        q_col_scale = prod;
      }
      if (weights_in_epilogue) {
        if (hipMemcpyAsync(qk_weight, w.query_norm_weight, static_cast<size_t>(D) * 2, hipMemcpyDeviceToDevice,
                           as_stream(stream)) != hipSuccess ||
            hipMemcpyAsync(qk_weight + D, w.key_norm_weight, static_cast<size_t>(D) * 2, hipMemcpyDeviceToDevice,
                           as_stream(stream)) != hipSuccess)
          return set_error(TAAC_ERR_LAUNCH, "%s: copy of the query / key norm weights failed", name);
      }
      if (planes)
        rc = norm_linear_qk_heads(cur, D, w.attn_norm_weight, eps, w.qkv_bias, pk_qkv, qkv, M, D, heads, T,
                                  weights_in_epilogue ? qk_weight : nullptr, rope_cos_sin, qk_norm ? qk_sumsq : nullptr,
                                  rows, n_rows, w.attn_norm_weight != nullptr, stream);
      else
        rc = taac_norm_linear_qk_fwd(cur, D, w.attn_norm_weight, eps, nullptr, w.qkv_bias, pk_qkv, qkv, 3 * D, M, D, heads,
                                     T, weights_in_epilogue ? qk_weight : nullptr, rope_cos_sin,
                                     qk_norm ? qk_sumsq : nullptr, rows, n_rows, nullptr, w.attn_norm_weight != nullptr,
                                     stream);
      if (rc != TAAC_OK) return rc;
      if (qk_norm) {
        if ((rc = taac_row_rstd(qk_sumsq, M, D, eps, qk_rstd, rows, n_rows, stream)) != TAAC_OK) return rc;
        q_scale = qk_rstd;
        k_scale = qk_rstd + M;
      }
    } else if (planes) {
      if ((rc = taac_norm_linear_heads_fwd(cur, D, w.attn_norm_weight, eps, w.qkv_bias, pk_qkv, qkv, dh, M, 3 * D, D, rows,
                                           n_rows, w.attn_norm_weight != nullptr, stream)) != TAAC_OK)
        return rc;
    } else if (fused) {
      if ((rc = taac_norm_linear_fwd(cur, D, w.attn_norm_weight, eps, nullptr, w.qkv_bias, pk_qkv, nullptr, 0, qkv,
                                     3 * D, M, 3 * D, D, rows, n_rows, nullptr, w.attn_norm_weight != nullptr,
                                     stream)) != TAAC_OK)
        return rc;
    } else {
      if ((rc = taac_rmsnorm_fwd(cur, w.attn_norm_weight, h, M, D, eps, TAAC_BF16, stream)) != TAAC_OK) return rc;
      if ((rc = taac_linear_bf16(h, D, w.qkv_weight, w.qkv_bias, nullptr, qkv, 3 * D, M, 3 * D, D, TAAC_EPI_NONE, 1,
                                 stream)) != TAAC_OK)
        return rc;
    }
    if (!fused && qk_prepare) {
      if ((rc = taac_qk_norm_rope_fwd(qkv, qkv + D, 3 * D, qkv, qkv + D, 3 * D, M, T, D, heads, w.query_norm_weight,
                                      w.key_norm_weight, eps, rope_cos_sin, nullptr, nullptr, TAAC_BF16, stream)) !=
          TAAC_OK)
        return rc;
    }
    if (planes) {
      if ((rc = taac_flash_attn_scaled_fwd(qkv, qkv + heads * plane_elems, qkv + 2 * heads * plane_elems, key_lengths,
                                           q_scale, k_scale, q_col_scale, h, B, heads, T, T, dh, plane_strides, plane_strides,
                                           plane_strides, plane_strides, 0, rows ? 2 : 1, TAAC_BF16, stream)) != TAAC_OK)
        return rc;
      if ((rc = attn_out_ffn_readout(h, D, dh, w.out_bias, pk_out, cur, D, w.ffn_norm_weight, eps, w.up_bias, w.down_bias,
                                     pk_ffn, x_out, D, M, D, F, rows, n_rows, ffn_folded,
                                     ride ? w_head : nullptr, ride ? token_dots : nullptr, stream)) != TAAC_OK)
        return rc;
      dots_ready = ride;
      cur = x_out;
      continue;
    }
    if ((rc = taac_flash_attn_scaled_fwd(qkv, qkv + D, qkv + 2 * D, key_lengths, q_scale, k_scale, q_col_scale, h, B,
                                         heads, T, T, dh, qkv_strides, qkv_strides, qkv_strides, o_strides, 0, rows ? 2 : 1,
                                         TAAC_BF16, stream)) != TAAC_OK)
      return rc;
    if (fused && !split_out_ffn) {
      // out projection + residual and the whole feed-forward half in one kernel; the stream between them stays on chip
      if ((rc = attn_out_ffn_readout(h, D, 0, w.out_bias, pk_out, cur, D, w.ffn_norm_weight, eps, w.up_bias, w.down_bias,
                                     pk_ffn, x_out, D, M, D, F, rows, n_rows, ffn_folded,
                                     ride ? w_head : nullptr, ride ? token_dots : nullptr, stream)) != TAAC_OK)
        return rc;
      dots_ready = ride;
    } else if (fused) {
      if ((rc = taac_norm_linear_fwd(h, D, nullptr, eps, nullptr, w.out_bias, pk_out, cur, D, x, D, M, D, D, rows,
                                     n_rows, nullptr, 0, stream)) != TAAC_OK)
        return rc;
      // feed-forward half: RMSNorm -> up -> SiLU-gate -> down -> + residual in one kernel
      if ((rc = taac_swiglu_ffn_fwd(x, D, w.ffn_norm_weight, eps, nullptr, w.up_bias, nullptr, w.down_bias, pk_ffn, x,
                                    D, x_out, D, M, D, F, 1, rows, n_rows, ffn_folded, stream)) != TAAC_OK)
        return rc;
    } else {
      if ((rc = taac_linear_bf16(h, D, w.out_weight, w.out_bias, cur, x, D, M, D, D, TAAC_EPI_RESIDUAL, 1, stream)) !=
          TAAC_OK)
        return rc;
      if ((rc = taac_rmsnorm_fwd(x, w.ffn_norm_weight, h, M, D, eps, TAAC_BF16, stream)) != TAAC_OK) return rc;
      if ((rc = taac_linear_bf16(h, D, w.up_weight, w.up_bias, nullptr, g, F, M, 2 * F, D, TAAC_EPI_SWIGLU, 1,
                                 stream)) != TAAC_OK)
        return rc;
      if ((rc = taac_linear_bf16(g, F, w.down_weight, w.down_bias, x, x_out, D, M, D, F, TAAC_EPI_RESIDUAL, 1,
                                 stream)) != TAAC_OK)
        return rc;
    }
    cur = x_out;
  }
  if (rows != nullptr && hidden_out != nullptr) {
    // The padded positions of the returned hidden state were never written: define them as zeros.
    const int64_t pieces = static_cast<int64_t>(T) * (D / 8);
    hipLaunchKernelGGL(zero_padded_rows_kernel, dim3(static_cast<uint32_t>((pieces + kBlock - 1) / kBlock), B),
                       dim3(kBlock), 0, as_stream(stream), static_cast<bf16_t*>(hidden_out), key_lengths, T, D);
    if ((rc = check_launch(name)) != TAAC_OK) return rc;
  }
  if (n_blocks == 0 && hidden_out != nullptr) {
    if (hipMemcpyAsync(hidden_out, emb, static_cast<size_t>(M) * D * 2, hipMemcpyDeviceToDevice, as_stream(stream)) !=
        hipSuccess)
      return set_error(TAAC_ERR_LAUNCH, "%s: copy of the embeddings failed", name);
  }
  if (dots_ready) {  // the last block's kernel left every token's dot product with the head weight behind
    const int per = kBlock / kWave;
    hipLaunchKernelGGL(token_dots_head_kernel, dim3((B + per - 1) / per), dim3(kBlock), 0, as_stream(stream), token_dots,
                       key_lengths, static_cast<const bf16_t*>(b_head), p, B, T);
    return check_launch(name);
  }
  return taac_masked_mean_head(cur, key_lengths, w_head, b_head, p, B, T, D, stream);
}

extern "C" int taac_front_rows(const int32_t* rows, const int32_t* n_rows, int32_t B, int32_t T, int32_t* front_rows,
                               int32_t* lengths, void* stream) {
  using namespace taac;
  const char* name = "taac_front_rows";
  if (B < 0 || T < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (static_cast<int64_t>(B) * T > 0x7fffffffLL - B - 1)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: B * T must fit 32-bit row numbers", name);
  if (B == 0) return TAAC_OK;
  if (!rows || !n_rows || !lengths || (T > 0 && !front_rows)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int64_t threads = static_cast<int64_t>(B) * T > B ? static_cast<int64_t>(B) * T : B;
  hipLaunchKernelGGL(front_rows_kernel, dim3(static_cast<uint32_t>((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                     as_stream(stream), rows, n_rows, B, T, front_rows, lengths);
  return check_launch(name);
}

extern "C" int taac_mask_front_bits(const uint32_t* struct_bits, int32_t T, const int32_t* rows, int32_t B,
                                    uint32_t* out_bits, void* stream) {
  using namespace taac;
  const char* name = "taac_mask_front_bits";
  if (B < 0 || T < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: bad dimensions", name);
  if (T > 4096) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 4096 tokens per sample", name);
  if (static_cast<int64_t>(B) * T > 0x7fffffffLL - B - 1)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: B * T must fit 32-bit row numbers", name);
  if (B == 0 || T == 0) return TAAC_OK;
  if (!struct_bits || !rows || !out_bits) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int64_t blocks = static_cast<int64_t>(B) * ((T + kFrontRowsPerBlock - 1) / kFrontRowsPerBlock);
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many rows", name);
  hipLaunchKernelGGL(mask_front_bits_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, as_stream(stream),
                     struct_bits, T, rows, B, out_bits);
  return check_launch(name);
}
