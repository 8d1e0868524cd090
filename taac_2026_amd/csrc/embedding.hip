// Multi-hot embedding lookup with mean pooling for gfx950: out[b, :] = mean over the non-padding ids of bag b of
// weight[id, :], id 0 = padding, an all-padding bag gives zeros (F.embedding_bag(values, weight, mode="mean",
// padding_idx=0), accelerators/embedding/embedding_bag.py:82-83).
//
// HBM-bound gather: a bag is owned by G consecutive lanes, each holding NV 16-byte pieces of the embedding row, so a
// table row is fetched as one contiguous run of 16-byte requests and the output row is written once. The ids of a bag
// are read four at a time and the (up to four) rows they name are requested before any of them is accumulated, fp32
// accumulation, one rounding.
#include "common.h"

namespace taac {
namespace {

constexpr int kBlock = 256;

template <typename T>
struct Piece;  // one 16-byte piece of a row
template <>
struct Piece<float> {
  static constexpr int N = 4;
  typedef f32x4 vec;
};
template <>
struct Piece<bf16_t> {
  static constexpr int N = 8;
  typedef bf16x8 vec;
};
template <>
struct Piece<f16_t> {
  static constexpr int N = 8;
  typedef f16x8 vec;
};

template <typename T, typename I, int G, int NV>
__global__ __launch_bounds__(kBlock) void embedding_bag_mean_kernel(const T* __restrict__ weight, int64_t num_embeddings,
                                                                     int emb_dim, const I* __restrict__ values,
                                                                     int64_t bags, int bag_size, T* __restrict__ out,
                                                                     int32_t* __restrict__ invalid_count) {
  typedef typename Piece<T>::vec vec_t;
  constexpr int N = Piece<T>::N;
  constexpr int GPB = kBlock / G;
  const int lane = threadIdx.x % G;
  const int64_t bag = static_cast<int64_t>(blockIdx.x) * GPB + threadIdx.x / G;
  if (bag >= bags) return;
  const int nvec = emb_dim / N;
  const I* ids = values + bag * bag_size;
  float acc[NV][N];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < N; ++e) acc[i][e] = 0.f;
  int count = 0, invalid = 0;
  for (int j0 = 0; j0 < bag_size; j0 += 4) {
    int64_t id[4];
    bool use[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      id[j] = j0 + j < bag_size ? static_cast<int64_t>(ids[j0 + j]) : 0;
      use[j] = id[j] > 0 && id[j] < num_embeddings;
      invalid += (id[j] < 0 || id[j] >= num_embeddings) ? 1 : 0;
      count += use[j] ? 1 : 0;
    }
    vec_t piece[4][NV];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lane + i * G;
        if (use[j] && v < nvec) piece[j][i] = *reinterpret_cast<const vec_t*>(weight + id[j] * emb_dim + v * N);
      }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lane + i * G;
        if (use[j] && v < nvec) {
#pragma unroll
          for (int e = 0; e < N; ++e) acc[i][e] += static_cast<float>(piece[j][i][e]);
        }
      }
  }
  const float inv = 1.0f / static_cast<float>(count > 0 ? count : 1);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + i * G;
    if (v < nvec) {
      vec_t o;
#pragma unroll
      for (int e = 0; e < N; ++e) o[e] = static_cast<T>(acc[i][e] * inv);
      __builtin_nontemporal_store(o, reinterpret_cast<vec_t*>(out + bag * emb_dim + v * N));
    }
  }
  if (invalid_count != nullptr && lane == 0 && invalid > 0) atomicAdd(invalid_count, invalid);
}

// Rows that are not a whole number of 16-byte pieces, or unaligned tables: one lane per element.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void embedding_bag_mean_generic_kernel(const T* __restrict__ weight,
                                                                             int64_t num_embeddings, int emb_dim,
                                                                             const I* __restrict__ values, int64_t bags,
                                                                             int bag_size, T* __restrict__ out,
                                                                             int32_t* __restrict__ invalid_count) {
  const int64_t bag = blockIdx.x;
  const I* ids = values + bag * bag_size;
  for (int c = threadIdx.x; c < emb_dim; c += kBlock) {
    float acc = 0.f;
    int count = 0, invalid = 0;
    for (int j = 0; j < bag_size; ++j) {
      const int64_t id = static_cast<int64_t>(ids[j]);
      if (id > 0 && id < num_embeddings) {
        acc += static_cast<float>(weight[id * emb_dim + c]);
        ++count;
      } else if (id != 0) {
        ++invalid;
      }
    }
    out[bag * emb_dim + c] = static_cast<T>(acc / static_cast<float>(count > 0 ? count : 1));
    if (invalid_count != nullptr && c == 0 && invalid > 0) atomicAdd(invalid_count, invalid);
  }
}

template <typename T, typename I, int G, int NV>
void launch_bag(const T* w, int64_t n, int e, const I* v, int64_t bags, int bag_size, T* out, int32_t* invalid,
                hipStream_t s) {
  constexpr int GPB = kBlock / G;
  hipLaunchKernelGGL((embedding_bag_mean_kernel<T, I, G, NV>), dim3(static_cast<uint32_t>((bags + GPB - 1) / GPB)),
                     dim3(kBlock), 0, s, w, n, e, v, bags, bag_size, out, invalid);
}

template <typename T, typename I>
int dispatch_bag(const void* weight, int64_t n, int e, const void* values, int64_t bags, int bag_size, void* out,
                 int32_t* invalid, hipStream_t s) {
  const T* w = static_cast<const T*>(weight);
  const I* v = static_cast<const I*>(values);
  T* o = static_cast<T*>(out);
  constexpr int N = Piece<T>::N;
  const int nvec = e / N;
  if (e % N != 0 || !aligned16(w) || !aligned16(o) || nvec > 64 * 8) {
    hipLaunchKernelGGL((embedding_bag_mean_generic_kernel<T, I>), dim3(static_cast<uint32_t>(bags)), dim3(kBlock), 0, s, w,
                       n, e, v, bags, bag_size, o, invalid);
    return TAAC_OK;
  }
#define TAAC_BAG_CASE(G, NV)                                          \
  launch_bag<T, I, G, NV>(w, n, e, v, bags, bag_size, o, invalid, s); \
  return TAAC_OK;
  if (nvec <= 1) { TAAC_BAG_CASE(1, 1) }
  if (nvec <= 2) { TAAC_BAG_CASE(2, 1) }
  if (nvec <= 4) { TAAC_BAG_CASE(4, 1) }
  if (nvec <= 8) { TAAC_BAG_CASE(8, 1) }
  if (nvec <= 16) { TAAC_BAG_CASE(16, 1) }
  if (nvec <= 32) { TAAC_BAG_CASE(32, 1) }
  if (nvec <= 64) { TAAC_BAG_CASE(64, 1) }
  if (nvec <= 128) { TAAC_BAG_CASE(64, 2) }
  if (nvec <= 256) { TAAC_BAG_CASE(64, 4) }
  TAAC_BAG_CASE(64, 8)
#undef TAAC_BAG_CASE
}

// Backward of the mean: every valid id j of bag b receives grad_out[b, :] / max(count_b, 1) on row id of the table's
// gradient (accelerators/embedding/kernels/triton.py:105-150, tilelang.py:95-140). The sums are formed in fp32 with
// the hardware's float add-to-memory; rows named by several bags therefore add in an order that varies from launch to
// launch (last-bit differences), as in the reference's atomic adds. One bag per G lanes like the forward; each lane keeps
// its slice of the scaled gradient row in registers over the bag's ids.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void embedding_bag_mean_bwd_kernel(const I* __restrict__ values, int64_t bags,
                                                                         int bag_size, const T* __restrict__ grad_out,
                                                                         float* __restrict__ grad_sum,
                                                                         int64_t num_embeddings, int emb_dim, int lanes) {
  const int per_block = kBlock / lanes;
  const int lane = threadIdx.x % lanes;
  const int64_t bag = static_cast<int64_t>(blockIdx.x) * per_block + threadIdx.x / lanes;
  if (bag >= bags) return;
  const I* ids = values + bag * bag_size;
  int count = 0;
  for (int j = 0; j < bag_size; ++j) {
    const int64_t id = static_cast<int64_t>(ids[j]);
    count += (id > 0 && id < num_embeddings) ? 1 : 0;
  }
  if (count == 0) return;
  const float inv = 1.0f / static_cast<float>(count);
  for (int c0 = 0; c0 < emb_dim; c0 += 4 * lanes) {
    float g[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = c0 + e * lanes + lane;
      g[e] = c < emb_dim ? static_cast<float>(grad_out[bag * emb_dim + c]) * inv : 0.f;
    }
    for (int j = 0; j < bag_size; ++j) {
      const int64_t id = static_cast<int64_t>(ids[j]);
      if (id <= 0 || id >= num_embeddings) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int c = c0 + e * lanes + lane;
        if (c < emb_dim) unsafeAtomicAdd(grad_sum + id * emb_dim + c, g[e]);
      }
    }
  }
}

__global__ __launch_bounds__(kBlock) void clear_sums_kernel(float* __restrict__ sums, int64_t count) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  const int64_t quads = count / 4;
  f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < quads; i += stride)
    reinterpret_cast<f32x4*>(sums)[i] = zero;
  for (int64_t i = quads * 4 + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < count; i += stride) sums[i] = 0.f;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void round_sums_kernel(const float* __restrict__ sums, T* __restrict__ out,
                                                             int64_t count) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < count; i += stride)
    out[i] = static_cast<T>(sums[i]);
}

template <typename T, typename I>
void launch_bag_bwd(const void* values, int64_t bags, int bag_size, const void* grad_out, float* sums, int64_t n, int e,
                    hipStream_t s) {
  int lanes = 1;
  while (lanes < 64 && lanes * 4 < e) lanes *= 2;
  const int per_block = kBlock / lanes;
  hipLaunchKernelGGL((embedding_bag_mean_bwd_kernel<T, I>), dim3(static_cast<uint32_t>((bags + per_block - 1) / per_block)),
                     dim3(kBlock), 0, s, static_cast<const I*>(values), bags, bag_size, static_cast<const T*>(grad_out),
                     sums, n, e, lanes);
}

}  // namespace
}  // namespace taac

extern "C" int taac_embedding_bag_mean_fwd(const void* weight, int64_t num_embeddings, int32_t emb_dim,
                                           const void* values, int index_is_int64, int64_t bags, int32_t bag_size,
                                           void* out, int32_t* invalid_count, int dtype, void* stream) {
  using namespace taac;
  const char* name = "taac_embedding_bag_mean_fwd";
  if (num_embeddings <= 0 || emb_dim <= 0 || bags < 0 || bag_size < 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: num_embeddings, emb_dim > 0 and bags, bag_size >= 0 required", name);
  if (bags == 0) return TAAC_OK;
  if (!weight || !out || (bag_size > 0 && !values)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (bags > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: more than 2^31-1 bags", name);
  hipStream_t s = as_stream(stream);
  int rc;
#define TAAC_BAG_DTYPE(T)                                                                                             \
  rc = index_is_int64 ? dispatch_bag<T, int64_t>(weight, num_embeddings, emb_dim, values, bags, bag_size, out,        \
                                                 invalid_count, s)                                                     \
                      : dispatch_bag<T, int32_t>(weight, num_embeddings, emb_dim, values, bags, bag_size, out,        \
                                                 invalid_count, s)
  switch (dtype) {
    case TAAC_F32: TAAC_BAG_DTYPE(float); break;
    case TAAC_BF16: TAAC_BAG_DTYPE(bf16_t); break;
    case TAAC_F16: TAAC_BAG_DTYPE(f16_t); break;
    default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  }
#undef TAAC_BAG_DTYPE
  if (rc != TAAC_OK) return rc;
  return check_launch(name);
}

extern "C" int taac_embedding_bag_mean_bwd(const void* values, int index_is_int64, int64_t bags, int32_t bag_size,
                                           const void* grad_out, void* grad_weight, int64_t num_embeddings,
                                           int32_t emb_dim, void* workspace, int dtype, void* stream) {
  using namespace taac;
  const char* name = "taac_embedding_bag_mean_bwd";
  if (num_embeddings <= 0 || emb_dim <= 0 || bags < 0 || bag_size < 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: num_embeddings, emb_dim > 0 and bags, bag_size >= 0 required", name);
  if (dtype != TAAC_F32 && dtype != TAAC_BF16 && dtype != TAAC_F16)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  if (!grad_weight || (bags > 0 && (!grad_out || (bag_size > 0 && !values))))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (dtype != TAAC_F32 && !workspace)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: a 16-bit table gradient needs the fp32 workspace (num_embeddings * emb_dim floats)", name);
  if (bags > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: more than 2^31-1 bags", name);
  if ((reinterpret_cast<uintptr_t>(dtype == TAAC_F32 ? grad_weight : workspace) & 15) != 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the fp32 sums must be 16-byte aligned", name);
  hipStream_t s = as_stream(stream);
  float* sums = static_cast<float*>(dtype == TAAC_F32 ? grad_weight : workspace);
  const int64_t count = num_embeddings * emb_dim;
  const uint32_t wide = static_cast<uint32_t>(std::min<int64_t>((count / 4 + kBlock) / kBlock, 256 * 16));
  hipLaunchKernelGGL(clear_sums_kernel, dim3(wide), dim3(kBlock), 0, s, sums, count);
  if (bags > 0 && bag_size > 0) {
#define TAAC_BAG_BWD(T)                                                                                            \
  index_is_int64 ? launch_bag_bwd<T, int64_t>(values, bags, bag_size, grad_out, sums, num_embeddings, emb_dim, s) \
                 : launch_bag_bwd<T, int32_t>(values, bags, bag_size, grad_out, sums, num_embeddings, emb_dim, s)
    if (dtype == TAAC_F32) TAAC_BAG_BWD(float);
    else if (dtype == TAAC_BF16) TAAC_BAG_BWD(bf16_t);
    else TAAC_BAG_BWD(f16_t);
#undef TAAC_BAG_BWD
  }
  if (dtype != TAAC_F32) {
    const uint32_t blocks = static_cast<uint32_t>(std::min<int64_t>((count + kBlock - 1) / kBlock, 256 * 16));
    if (dtype == TAAC_BF16)
      hipLaunchKernelGGL((round_sums_kernel<bf16_t>), dim3(blocks), dim3(kBlock), 0, s, sums, static_cast<bf16_t*>(grad_weight), count);
    else
      hipLaunchKernelGGL((round_sums_kernel<f16_t>), dim3(blocks), dim3(kBlock), 0, s, sums, static_cast<f16_t*>(grad_weight), count);
  }
  return check_launch(name);
}
