// RMSNorm / LayerNorm forward for gfx950: single-pass row kernels.
//
// A row is owned by a group of G consecutive lanes of one wavefront (G = 1..64, a power of two). Each lane keeps
// NV 128-bit vectors of the row in registers, so x is read from HBM exactly once and y written exactly once;
// the reductions are wavefront shuffles inside the lane group and all arithmetic is fp32. Consecutive groups own
// consecutive rows, so a wavefront's loads and stores cover one contiguous span of memory.
//
// Arithmetic follows the reference's closed forms
//   RMSNorm:   y = x * rsqrt(mean(x^2) + eps) * w      (accelerators/normalization/rms_norm.py:71-73)
//   LayerNorm: y = (x - mean) * rsqrt(var + eps) * w + b, var from centred values
//                                                      (normalization/kernels/triton.py:224-247)
#include <mutex>

#include "common.h"

namespace taac {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxNV = 8;

template <typename T>
struct Pack;
template <>
struct Pack<float> {
  static constexpr int VEC = 4;
  typedef f32x4 vec;
  static __device__ __forceinline__ void unpack(const vec& v, float* f) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) f[i] = v[i];
  }
  static __device__ __forceinline__ vec pack(const float* f) {
    vec v;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = f[i];
    return v;
  }
};
template <>
struct Pack<bf16_t> {
  static constexpr int VEC = 8;
  typedef bf16x8 vec;
  static __device__ __forceinline__ void unpack(const vec& v, float* f) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) f[i] = static_cast<float>(v[i]);
  }
  static __device__ __forceinline__ vec pack(const float* f) {
    vec v;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = static_cast<bf16_t>(f[i]);
    return v;
  }
};
template <>
struct Pack<f16_t> {
  static constexpr int VEC = 8;
  typedef f16x8 vec;
  static __device__ __forceinline__ void unpack(const vec& v, float* f) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) f[i] = static_cast<float>(v[i]);
  }
  static __device__ __forceinline__ vec pack(const float* f) {
    vec v;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = static_cast<f16_t>(f[i]);
    return v;
  }
};

// One block = 256 / G lane groups, each group normalises R rows per launch slot.
template <typename T, int G, int NV, int R, bool LN>
__global__ __launch_bounds__(kBlock) void norm_rows_vec_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                               const T* __restrict__ b, T* __restrict__ y,
                                                               int64_t rows, int cols, int nvec, float eps) {
  typedef Pack<T> P;
  typedef typename P::vec vec_t;
  constexpr int VEC = P::VEC;
  constexpr int GPB = kBlock / G;  // lane groups (rows in flight) per block
  const int lane = threadIdx.x % G;
  const int gid = threadIdx.x / G;

  // Issue every load of this thread before touching the data: R * NV independent 128-bit loads in flight.
  vec_t raw[R][NV];
  bool row_ok[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = (static_cast<int64_t>(blockIdx.x) * R + r) * GPB + gid;
    row_ok[r] = row < rows;
    const vec_t* xr = reinterpret_cast<const vec_t*>(x + row * cols);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = lane + i * G;
      if (row_ok[r] && v < nvec) {
        raw[r][i] = __builtin_nontemporal_load(xr + v);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) raw[r][i][e] = 0;
      }
    }
  }

  float wf[NV][VEC];
  float bf[LN ? NV : 1][VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + i * G;
    if (v < nvec) {
      P::unpack(reinterpret_cast<const vec_t*>(w)[v], wf[i]);
      if (LN) P::unpack(reinterpret_cast<const vec_t*>(b)[v], bf[LN ? i : 0]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        wf[i][e] = 0.f;
        if (LN) bf[LN ? i : 0][e] = 0.f;
      }
    }
  }

  const float inv_cols = 1.0f / static_cast<float>(cols);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float xf[NV][VEC];
#pragma unroll
    for (int i = 0; i < NV; ++i) P::unpack(raw[r][i], xf[i]);

    float mean = 0.f;
    if (LN) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) s += xf[i][e];
      mean = group_sum<G>(s) * inv_cols;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const bool live = (lane + i * G) < nvec;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float c = LN ? (live ? xf[i][e] - mean : 0.f) : xf[i][e];
        ss += c * c;
      }
    }
    ss = group_sum<G>(ss);
    const float scale = rsqrtf(ss * inv_cols + eps);

    if (row_ok[r]) {
      const int64_t row = (static_cast<int64_t>(blockIdx.x) * R + r) * GPB + gid;
      vec_t* yr = reinterpret_cast<vec_t*>(y + row * cols);
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lane + i * G;
        if (v < nvec) {
          float of[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            if (LN)
              of[e] = (xf[i][e] - mean) * scale * wf[i][e] + bf[LN ? i : 0][e];
            else
              of[e] = xf[i][e] * scale * wf[i][e];
          }
          __builtin_nontemporal_store(P::pack(of), yr + v);
        }
      }
    }
  }
}

// Fallback for column counts that are not a whole number of 128-bit vectors, unaligned bases, or very long rows:
// one wavefront per row, element-wise loads; the second and third sweep of a row come from cache.
template <typename T, bool LN>
__global__ __launch_bounds__(kBlock) void norm_rows_generic_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                   const T* __restrict__ b, T* __restrict__ y,
                                                                   int64_t rows, int cols, float eps) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  const T* xr = x + row * cols;
  T* yr = y + row * cols;
  const float inv_cols = 1.0f / static_cast<float>(cols);
  float mean = 0.f;
  if (LN) {
    float s = 0.f;
    for (int c = lane; c < cols; c += kWave) s += static_cast<float>(xr[c]);
    mean = group_sum<kWave>(s) * inv_cols;
  }
  float ss = 0.f;
  for (int c = lane; c < cols; c += kWave) {
    const float d = static_cast<float>(xr[c]) - mean;
    ss += d * d;
  }
  ss = group_sum<kWave>(ss);
  const float scale = rsqrtf(ss * inv_cols + eps);
  for (int c = lane; c < cols; c += kWave) {
    const float xv = static_cast<float>(xr[c]);
    float o;
    if (LN)
      o = (xv - mean) * scale * static_cast<float>(w[c]) + static_cast<float>(b[c]);
    else
      o = xv * scale * static_cast<float>(w[c]);
    yr[c] = static_cast<T>(o);
  }
}

template <typename T, int G, int NV, bool LN>
void launch_vec(const T* x, const T* w, const T* b, T* y, int64_t rows, int cols, int nvec, float eps,
                hipStream_t s) {
  constexpr int R = (NV <= 2) ? 2 : 1;
  constexpr int GPB = kBlock / G;
  const int64_t rows_per_block = static_cast<int64_t>(GPB) * R;
  const int64_t grid = (rows + rows_per_block - 1) / rows_per_block;
  hipLaunchKernelGGL((norm_rows_vec_kernel<T, G, NV, R, LN>), dim3(static_cast<uint32_t>(grid)), dim3(kBlock), 0, s,
                     x, w, b, y, rows, cols, nvec, eps);
}

template <typename T, bool LN>
int dispatch(const void* xv, const void* wv, const void* bv, void* yv, int64_t rows, int cols, float eps,
             hipStream_t s) {
  const T* x = static_cast<const T*>(xv);
  const T* w = static_cast<const T*>(wv);
  const T* b = static_cast<const T*>(bv);
  T* y = static_cast<T*>(yv);
  constexpr int VEC = Pack<T>::VEC;
  const bool vec_ok = (cols % VEC == 0) && aligned16(x) && aligned16(y) && aligned16(w) && (!LN || aligned16(b)) &&
                      (cols / VEC) <= kWave * kMaxNV;
  if (!vec_ok) {
    const int64_t grid = (rows + (kBlock / kWave) - 1) / (kBlock / kWave);
    hipLaunchKernelGGL((norm_rows_generic_kernel<T, LN>), dim3(static_cast<uint32_t>(grid)), dim3(kBlock), 0, s, x, w,
                       b, y, rows, cols, eps);
    return TAAC_OK;
  }
  const int nvec = cols / VEC;
#define TAAC_NORM_CASE(G, NV)                                          \
  launch_vec<T, G, NV, LN>(x, w, b, y, rows, cols, nvec, eps, s);      \
  return TAAC_OK;
  if (nvec <= 1) { TAAC_NORM_CASE(1, 1) }
  if (nvec <= 2) { TAAC_NORM_CASE(2, 1) }
  if (nvec <= 4) { TAAC_NORM_CASE(4, 1) }
  if (nvec <= 8) { TAAC_NORM_CASE(8, 1) }
  if (nvec <= 16) { TAAC_NORM_CASE(16, 1) }
  if (nvec <= 32) { TAAC_NORM_CASE(32, 1) }
  if (nvec <= 64) { TAAC_NORM_CASE(64, 1) }
  if (nvec <= 128) { TAAC_NORM_CASE(64, 2) }
  if (nvec <= 256) { TAAC_NORM_CASE(64, 4) }
  TAAC_NORM_CASE(64, 8)
#undef TAAC_NORM_CASE
}

template <bool LN>
int norm_entry(const char* name, const void* x, const void* w, const void* b, void* y, int64_t rows, int32_t cols,
               float eps, int dtype, void* stream) {
  if (rows < 0 || cols <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows must be >= 0 and cols > 0", name);
  if (rows == 0) return TAAC_OK;
  if (!x || !w || !y || (LN && !b)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  const int64_t max_rows = static_cast<int64_t>(0x7fffffff) * 1;  // grid.x limit with >= 1 row per block
  if (rows > max_rows) return set_error(TAAC_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", name);
  hipStream_t s = as_stream(stream);
  int rc;
  switch (dtype) {
    case TAAC_F32: rc = dispatch<float, LN>(x, w, b, y, rows, cols, eps, s); break;
    case TAAC_BF16: rc = dispatch<bf16_t, LN>(x, w, b, y, rows, cols, eps, s); break;
    case TAAC_F16: rc = dispatch<f16_t, LN>(x, w, b, y, rows, cols, eps, s); break;
    default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  }
  if (rc != TAAC_OK) return rc;
  return check_launch(name);
}


// ---- backward ----------------------------------------------------------------------------------------------------------
//
// RMSNorm:   g = dy * w, x_hat = x * rstd:            dx = rstd * (g - x_hat * mean(g * x_hat)),           dw = sum_rows dy * x_hat
// LayerNorm: g = dy * w, x_hat = (x - mean) * rstd:   dx = rstd * (g - mean(g) - x_hat * mean(g * x_hat)), dw as above,
//                                                     db = sum_rows dy
// (normalization/kernels/triton.py:82-116, 276-320). The row statistics are recomputed from x, which the kernel reads
// anyway, so nothing has to be saved by the forward. One pass: x and dy read once, dx written once. A workgroup walks
// several row tiles and keeps its share of dw / db in registers; per workgroup one partial row is written
// (fixed order inside the workgroup, through LDS), and a second small kernel adds the partials in order: the result
// does not depend on scheduling.
template <typename T, int G, int NV, bool LN>
__global__ __launch_bounds__(kBlock) void norm_bwd_rows_vec_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                    const T* __restrict__ dy, T* __restrict__ dx,
                                                                    float* __restrict__ partial, int64_t rows, int cols,
                                                                    int nvec, float eps) {
  typedef Pack<T> P;
  typedef typename P::vec vec_t;
  constexpr int VEC = P::VEC;
  constexpr int GPB = kBlock / G;
  __shared__ float red[GPB][G * VEC];
  const int lane = threadIdx.x % G;
  const int gid = threadIdx.x / G;
  const float inv_cols = 1.0f / static_cast<float>(cols);

  float wf[NV][VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + i * G;
    if (v < nvec) {
      P::unpack(reinterpret_cast<const vec_t*>(w)[v], wf[i]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) wf[i][e] = 0.f;
    }
  }
  float dwacc[NV][VEC], dbacc[LN ? NV : 1][VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      dwacc[i][e] = 0.f;
      if (LN) dbacc[LN ? i : 0][e] = 0.f;
    }

  constexpr int R = NV == 1 ? 4 : (NV == 2 ? 2 : 1);  // rows in flight per lane group
  for (int64_t row0 = static_cast<int64_t>(blockIdx.x) * (GPB * R); row0 < rows;
       row0 += static_cast<int64_t>(gridDim.x) * (GPB * R)) {
    // every load of the R rows is issued before any of them is used
    vec_t xr[R][NV], gr[R][NV];
    bool ok[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = row0 + r * GPB + gid;
      ok[r] = row < rows;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lane + i * G;
        if (ok[r] && v < nvec) {
          xr[r][i] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(x + row * cols) + v);
          gr[r][i] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(dy + row * cols) + v);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            xr[r][i][e] = 0;
            gr[r][i][e] = 0;
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = row0 + r * GPB + gid;
      float xf[NV][VEC], gf[NV][VEC];
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        P::unpack(xr[r][i], xf[i]);
        P::unpack(gr[r][i], gf[i]);
      }
      float mean = 0.f;
      if (LN) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
          for (int e = 0; e < VEC; ++e) sum += xf[i][e];
        mean = group_sum<G>(sum) * inv_cols;
      }
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const bool live = (lane + i * G) < nvec;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          xf[i][e] = LN ? (live ? xf[i][e] - mean : 0.f) : xf[i][e];  // centred from here on
          ss += xf[i][e] * xf[i][e];
        }
      }
      const float rstd = rsqrtf(group_sum<G>(ss) * inv_cols + eps);
      float sg = 0.f, sgx = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          xf[i][e] *= rstd;  // x_hat
          const float g = gf[i][e] * wf[i][e];
          sg += g;
          sgx += g * xf[i][e];
        }
      const float mean_gx = group_sum<G>(sgx) * inv_cols;
      const float mean_g = LN ? group_sum<G>(sg) * inv_cols : 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = lane + i * G;
        float of[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          of[e] = rstd * (gf[i][e] * wf[i][e] - mean_g - xf[i][e] * mean_gx);
          dwacc[i][e] += gf[i][e] * xf[i][e];  // rows beyond the end contribute zeros
          if (LN) dbacc[LN ? i : 0][e] += gf[i][e];
        }
        if (ok[r] && v < nvec) __builtin_nontemporal_store(P::pack(of), reinterpret_cast<vec_t*>(dx + row * cols) + v);
      }
    }
  }

  // Partial row of this workgroup: for every vector index the GPB lane groups meet in LDS and one thread per column adds
  // them in group order.
  float* out_w = partial + static_cast<int64_t>(blockIdx.x) * cols * (LN ? 2 : 1);
#pragma unroll
  for (int pass = 0; pass < (LN ? 2 : 1); ++pass) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      __syncthreads();
#pragma unroll
      for (int e = 0; e < VEC; ++e) red[gid][lane * VEC + e] = pass == 0 ? dwacc[i][e] : dbacc[LN ? i : 0][e];
      __syncthreads();
      for (int t = threadIdx.x; t < G * VEC; t += kBlock) {
        float sum = 0.f;
#pragma unroll
        for (int g = 0; g < GPB; ++g) sum += red[g][t];
        // column of element e of vector lane + i * G is (lane + i * G) * VEC + e = i * G * VEC + t
        const int col = i * G * VEC + t;
        if (col < cols) out_w[pass * cols + col] = sum;
      }
    }
  }
}

// dw[c] (and db[c]) = sum over the workgroups' partial rows in a fixed order: a workgroup owns 16 columns, thread
// (column, slice) adds the partial rows slice, slice + 16, ... and the 16 slice sums of a column are added in slice order.
template <typename T>
__global__ __launch_bounds__(kBlock) void norm_bwd_reduce_kernel(const float* __restrict__ partial, int nblocks, int cols,
                                                                  int parts, T* __restrict__ dw, T* __restrict__ db) {
  constexpr int CPB = 16, SLICES = kBlock / CPB;
  __shared__ float red[SLICES][CPB];
  const int cl = threadIdx.x % CPB, slice = threadIdx.x / CPB;
  const int c = blockIdx.x * CPB + cl;
  for (int part = 0; part < parts; ++part) {
    float sum = 0.f;
    if (c < cols) {
#pragma unroll 4
      for (int b = slice; b < nblocks; b += SLICES) sum += partial[(static_cast<int64_t>(b) * parts + part) * cols + c];
    }
    __syncthreads();
    red[slice][cl] = sum;
    __syncthreads();
    if (slice == 0 && c < cols) {
      float total = 0.f;
#pragma unroll
      for (int sl = 0; sl < SLICES; ++sl) total += red[sl][cl];
      T* dst = part == 0 ? dw : db;
      if (dst != nullptr) dst[c] = static_cast<T>(total);
    }
  }
}

// Sum over the workgroup of up to three values at once (wavefront shuffles, then one LDS round over the wavefronts);
// every thread gets the totals. `red` is reused by consecutive calls: the leading barrier protects the previous round.
template <int N>
__device__ __forceinline__ void block_sum(float (&v)[N], float (*red)[kBlock / kWave]) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = group_sum<kWave>(v[i]);
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < N; ++i) red[i][wave] = v[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) total += red[i][w];
    v[i] = total;
  }
}

// Backward for shapes the vector kernel does not take (columns that are not whole 128-bit vectors, unaligned bases,
// rows longer than its register budget): one workgroup per row at a time, thread t owns columns t, t + 256, ...; the
// row is swept four times (mean, variance, the two projections, the result), sweeps after the first come from cache.
// The workgroup's partial row of dw / db lives in the workspace and is updated in place by the thread that owns the
// column, in row order, so the result is reproducible as in the vector kernel.
template <typename T, bool LN>
__global__ __launch_bounds__(kBlock) void norm_bwd_rows_generic_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                        const T* __restrict__ dy, T* __restrict__ dx,
                                                                        float* __restrict__ partial, int64_t rows,
                                                                        int cols, float eps) {
  __shared__ float red[2][kBlock / kWave];
  const int tid = threadIdx.x;
  const float inv_cols = 1.0f / static_cast<float>(cols);
  float* out_w = partial + static_cast<int64_t>(blockIdx.x) * cols * (LN ? 2 : 1);
  for (int c = tid; c < cols; c += kBlock) {
    out_w[c] = 0.f;
    if (LN) out_w[cols + c] = 0.f;
  }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* xr = x + row * cols;
    const T* gr = dy + row * cols;
    T* dr = dx + row * cols;
    float mean = 0.f;
    if (LN) {
      float s[1] = {0.f};
      for (int c = tid; c < cols; c += kBlock) s[0] += static_cast<float>(xr[c]);
      block_sum<1>(s, red);
      mean = s[0] * inv_cols;
    }
    float ss[1] = {0.f};
    for (int c = tid; c < cols; c += kBlock) {
      const float d = static_cast<float>(xr[c]) - mean;
      ss[0] += d * d;
    }
    block_sum<1>(ss, red);
    const float rstd = rsqrtf(ss[0] * inv_cols + eps);
    float proj[2] = {0.f, 0.f};  // sum of g, sum of g * x_hat
    for (int c = tid; c < cols; c += kBlock) {
      const float g = static_cast<float>(gr[c]) * static_cast<float>(w[c]);
      proj[0] += g;
      proj[1] += g * ((static_cast<float>(xr[c]) - mean) * rstd);
    }
    block_sum<2>(proj, red);
    const float mean_g = LN ? proj[0] * inv_cols : 0.f;
    const float mean_gx = proj[1] * inv_cols;
    for (int c = tid; c < cols; c += kBlock) {
      const float gy = static_cast<float>(gr[c]);
      const float xh = (static_cast<float>(xr[c]) - mean) * rstd;
      dr[c] = static_cast<T>(rstd * (gy * static_cast<float>(w[c]) - mean_g - xh * mean_gx));
      out_w[c] += gy * xh;
      if (LN) out_w[cols + c] += gy;
    }
  }
}

constexpr int kBwdMaxBlocks = 1024;

template <typename T, bool LN>
int dispatch_bwd(const void* xv, const void* wv, const void* dyv, void* dxv, void* dwv, void* dbv, float* workspace,
                 int64_t workspace_floats, int64_t rows, int cols, float eps, hipStream_t s, const char* name) {
  const T* x = static_cast<const T*>(xv);
  const T* w = static_cast<const T*>(wv);
  const T* dy = static_cast<const T*>(dyv);
  T* dx = static_cast<T*>(dxv);
  constexpr int VEC = Pack<T>::VEC;
  const int parts = LN ? 2 : 1;
  if (cols % VEC != 0 || !aligned16(x) || !aligned16(dy) || !aligned16(dx) || !aligned16(w) || cols / VEC > kWave * 4) {
    // generic route: one workgroup per row at a time
    const int64_t nb = rows < kBwdMaxBlocks ? rows : kBwdMaxBlocks;
    if (workspace == nullptr || workspace_floats < nb * parts * cols)
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: workspace must hold %lld floats", name, (long long)(nb * parts * cols));
    if (rows > 0)
      hipLaunchKernelGGL((norm_bwd_rows_generic_kernel<T, LN>), dim3(static_cast<uint32_t>(nb)), dim3(kBlock), 0, s, x, w,
                         dy, dx, workspace, rows, cols, eps);
    hipLaunchKernelGGL((norm_bwd_reduce_kernel<T>), dim3((cols + 15) / 16), dim3(kBlock), 0, s, workspace,
                       static_cast<int>(nb), cols, parts, static_cast<T*>(dwv), static_cast<T*>(dbv));
    return TAAC_OK;
  }
  const int nvec = cols / VEC;
  int G = 1;
  while (G < nvec && G < kWave) G *= 2;
  const int rows_in_flight = nvec <= kWave ? 4 : (nvec <= 2 * kWave ? 2 : 1);  // R of the kernel
  const int gpb = (kBlock / G) * rows_in_flight;
  int64_t nblocks = (rows + gpb - 1) / gpb;
  if (nblocks > kBwdMaxBlocks) nblocks = kBwdMaxBlocks;
  if (workspace == nullptr || workspace_floats < nblocks * parts * cols)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: workspace must hold %lld floats", name,
                     (long long)(nblocks * parts * cols));
#define TAAC_BWD_CASE(GG, NV)                                                                                           \
  hipLaunchKernelGGL((norm_bwd_rows_vec_kernel<T, GG, NV, LN>), dim3(static_cast<uint32_t>(nblocks)), dim3(kBlock), 0, s, \
                     x, w, dy, dx, workspace, rows, cols, nvec, eps);                                                    \
  break;
  if (rows > 0) switch (G) {
    case 1: TAAC_BWD_CASE(1, 1)
    case 2: TAAC_BWD_CASE(2, 1)
    case 4: TAAC_BWD_CASE(4, 1)
    case 8: TAAC_BWD_CASE(8, 1)
    case 16: TAAC_BWD_CASE(16, 1)
    case 32: TAAC_BWD_CASE(32, 1)
    default:
      if (nvec <= 64) {
        TAAC_BWD_CASE(64, 1)
      } else if (nvec <= 128) {
        TAAC_BWD_CASE(64, 2)
      } else {
        TAAC_BWD_CASE(64, 4)
      }
  }
#undef TAAC_BWD_CASE
  hipLaunchKernelGGL((norm_bwd_reduce_kernel<T>), dim3((cols + 15) / 16), dim3(kBlock), 0, s, workspace,
                     static_cast<int>(nblocks), cols, parts, static_cast<T*>(dwv), static_cast<T*>(dbv));
  return TAAC_OK;
}

template <bool LN>
int norm_bwd_entry(const char* name, const void* x, const void* w, const void* dy, void* dx, void* dw, void* db,
                   float* workspace, int64_t workspace_floats, int64_t rows, int32_t cols, float eps, int dtype,
                   void* stream) {
  if (rows < 0 || cols <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows must be >= 0 and cols > 0", name);
  if (!x || !w || !dy || !dx) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  hipStream_t s = as_stream(stream);
  int rc;
  switch (dtype) {
    case TAAC_F32: rc = dispatch_bwd<float, LN>(x, w, dy, dx, dw, db, workspace, workspace_floats, rows, cols, eps, s, name); break;
    case TAAC_BF16: rc = dispatch_bwd<bf16_t, LN>(x, w, dy, dx, dw, db, workspace, workspace_floats, rows, cols, eps, s, name); break;
    case TAAC_F16: rc = dispatch_bwd<f16_t, LN>(x, w, dy, dx, dw, db, workspace, workspace_floats, rows, cols, eps, s, name); break;
    default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  }
  if (rc != TAAC_OK) return rc;
  return check_launch(name);
}

// ---- query / key RMSNorm + rotary embedding ---------------------------------------------------------------------------
//
// Work unit u = (token slot u / 2, which = u % 2): the query (0) or key (1) row of one token; the two rows of a token
// go to neighbouring lane groups, so with the packed [q | k | v] layout a wavefront reads one contiguous span. A row is
// held in registers between the statistic and the scaling, so q and k are read once and written once. The rotary
// table holds (cos, sin) of feature pair i of a head at [position][2i], [position][2i + 1] in the storage dtype, i.e.
// a lane that owns features d .. d + VEC - 1 of a head reads the VEC table entries at [position][d ..].
struct QkParams {
  const void* q;
  const void* k;
  void* q_out;
  void* k_out;
  const void* q_weight;
  const void* k_weight;
  const void* cos_sin;
  const int32_t* row_index;
  const int32_t* n_rows;
  int64_t ld_in, ld_out, rows;
  int32_t tokens_per_sample, d_model, head_dim, nvec;
  float eps;
};

template <typename T, int G, int NV, int R, bool NORM, bool ROPE>
__global__ __launch_bounds__(kBlock) void qk_norm_rope_kernel(const QkParams p) {
  typedef Pack<T> P;
  typedef typename P::vec vec_t;
  constexpr int VEC = P::VEC;
  constexpr int GPB = kBlock / G;
  const int lane = threadIdx.x % G;
  const int gid = threadIdx.x / G;
  const int64_t count = p.n_rows ? static_cast<int64_t>(*p.n_rows) : p.rows;

  vec_t raw[R][NV];
  vec_t table[ROPE ? R : 1][ROPE ? NV : 1];
  bool live[R];
  int64_t row[R];
  int which[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t unit = (static_cast<int64_t>(blockIdx.x) * R + r) * GPB + gid;
    const int64_t slot = unit >> 1;
    which[r] = static_cast<int>(unit & 1);
    live[r] = slot < count;
    row[r] = live[r] ? (p.row_index ? static_cast<int64_t>(p.row_index[slot]) : slot) : 0;
    const T* src = static_cast<const T*>(which[r] ? p.k : p.q) + row[r] * p.ld_in;
    const int pos = static_cast<int>(row[r] % p.tokens_per_sample);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = lane + i * G;
      if (live[r] && v < p.nvec) {
        raw[r][i] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(src + v * VEC));
        if (ROPE) {
          const int d = (v * VEC) % p.head_dim;
          table[ROPE ? r : 0][ROPE ? i : 0] = *reinterpret_cast<const vec_t*>(
              static_cast<const T*>(p.cos_sin) + static_cast<int64_t>(pos) * p.head_dim + d);
        }
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) raw[r][i][e] = 0;
      }
    }
  }

  const float inv_cols = 1.0f / static_cast<float>(p.d_model);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float xf[NV][VEC];
#pragma unroll
    for (int i = 0; i < NV; ++i) P::unpack(raw[r][i], xf[i]);
    float scale = 1.0f;
    if (NORM) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) ss += xf[i][e] * xf[i][e];
      ss = group_sum<G>(ss);
      scale = rsqrtf(ss * inv_cols + p.eps);
    }
    if (!live[r]) continue;
    T* dst = static_cast<T*>(which[r] ? p.k_out : p.q_out) + row[r] * p.ld_out;
    const T* w = static_cast<const T*>(which[r] ? p.k_weight : p.q_weight);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = lane + i * G;
      if (v >= p.nvec) continue;
      float of[VEC];
      if (NORM) {
        float wf[VEC];
        P::unpack(*reinterpret_cast<const vec_t*>(w + v * VEC), wf);
#pragma unroll
        for (int e = 0; e < VEC; ++e) of[e] = xf[i][e] * scale * wf[e];
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) of[e] = xf[i][e];
      }
      if (ROPE) {
        float cs[VEC];
        P::unpack(table[ROPE ? r : 0][ROPE ? i : 0], cs);
#pragma unroll
        for (int e = 0; e < VEC; e += 2) {
          const float even = of[e], odd = of[e + 1];
          of[e] = even * cs[e] - odd * cs[e + 1];
          of[e + 1] = even * cs[e + 1] + odd * cs[e];
        }
      }
      __builtin_nontemporal_store(P::pack(of), reinterpret_cast<vec_t*>(dst + v * VEC));
    }
  }
}

template <typename T, int G, int NV>
void launch_qk(const QkParams& p, bool norm, bool rope, hipStream_t s) {
  constexpr int R = NV <= 2 ? 4 : 2;
  constexpr int GPB = kBlock / G;
  const int64_t units = 2 * p.rows;
  const int64_t per_block = static_cast<int64_t>(GPB) * R;
  const dim3 grid(static_cast<uint32_t>((units + per_block - 1) / per_block));
  if (norm && rope)
    hipLaunchKernelGGL((qk_norm_rope_kernel<T, G, NV, R, true, true>), grid, dim3(kBlock), 0, s, p);
  else if (norm)
    hipLaunchKernelGGL((qk_norm_rope_kernel<T, G, NV, R, true, false>), grid, dim3(kBlock), 0, s, p);
  else
    hipLaunchKernelGGL((qk_norm_rope_kernel<T, G, NV, R, false, true>), grid, dim3(kBlock), 0, s, p);
}

template <typename T>
int dispatch_qk(QkParams p, bool norm, bool rope, hipStream_t s, const char* name) {
  constexpr int VEC = Pack<T>::VEC;
  const bool ok = p.d_model % VEC == 0 && p.ld_in % VEC == 0 && p.ld_out % VEC == 0 && aligned16(p.q) &&
                  aligned16(p.k) && aligned16(p.q_out) && aligned16(p.k_out) &&
                  (!norm || (aligned16(p.q_weight) && aligned16(p.k_weight))) &&
                  (!rope || (p.head_dim % VEC == 0 && aligned16(p.cos_sin)));
  if (!ok)
    return set_error(TAAC_ERR_UNSUPPORTED,
                     "%s: d_model, head_dim (with a rotary table) and the row strides must be multiples of %d elements "
                     "and every pointer 16-byte aligned",
                     name, VEC);
  p.nvec = p.d_model / VEC;
  if (p.nvec > kWave * kMaxNV) return set_error(TAAC_ERR_UNSUPPORTED, "%s: d_model above %d", name, kWave * kMaxNV * VEC);
#define TAAC_QK_CASE(G, NV)               \
  launch_qk<T, G, NV>(p, norm, rope, s);  \
  return TAAC_OK;
  if (p.nvec <= 4) { TAAC_QK_CASE(4, 1) }
  if (p.nvec <= 8) { TAAC_QK_CASE(8, 1) }
  if (p.nvec <= 16) { TAAC_QK_CASE(16, 1) }
  if (p.nvec <= 32) { TAAC_QK_CASE(32, 1) }
  if (p.nvec <= 64) { TAAC_QK_CASE(64, 1) }
  if (p.nvec <= 128) { TAAC_QK_CASE(64, 2) }
  if (p.nvec <= 256) { TAAC_QK_CASE(64, 4) }
  TAAC_QK_CASE(64, 8)
#undef TAAC_QK_CASE
}

}  // namespace
}  // namespace taac

extern "C" int taac_rmsnorm_fwd(const void* x, const void* w, void* y, int64_t rows, int32_t cols, float eps,
                                int dtype, void* stream) {
  return taac::norm_entry<false>("taac_rmsnorm_fwd", x, w, nullptr, y, rows, cols, eps, dtype, stream);
}

extern "C" int taac_layernorm_fwd(const void* x, const void* w, const void* b, void* y, int64_t rows, int32_t cols,
                                  float eps, int dtype, void* stream) {
  return taac::norm_entry<true>("taac_layernorm_fwd", x, w, b, y, rows, cols, eps, dtype, stream);
}

extern "C" int taac_qk_norm_rope_fwd(const void* q, const void* k, int64_t ld_in, void* q_out, void* k_out,
                                     int64_t ld_out, int64_t rows, int32_t tokens_per_sample, int32_t d_model,
                                     int32_t num_heads, const void* q_weight, const void* k_weight, float eps,
                                     const void* cos_sin, const int32_t* row_index, const int32_t* n_rows, int dtype,
                                     void* stream) {
  using namespace taac;
  const char* name = "taac_qk_norm_rope_fwd";
  if (rows < 0 || d_model <= 0 || num_heads <= 0 || tokens_per_sample <= 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows >= 0 and d_model, num_heads, tokens_per_sample > 0 required", name);
  if (d_model % num_heads != 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: d_model must be divisible by num_heads", name);
  if (rows == 0) return TAAC_OK;
  if (!q || !k || !q_out || !k_out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if ((q_weight == nullptr) != (k_weight == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: query and key norm weights come together", name);
  if (!q_weight && !cos_sin) return set_error(TAAC_ERR_INVALID_VALUE, "%s: neither norm weights nor a rotary table", name);
  if (ld_in < d_model || ld_out < d_model) return set_error(TAAC_ERR_INVALID_VALUE, "%s: row stride below d_model", name);
  if ((row_index == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row_index and n_rows come together", name);
  if (rows > 0x3fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: more than 2^30-1 rows", name);
  QkParams p{};
  p.q = q;
  p.k = k;
  p.q_out = q_out;
  p.k_out = k_out;
  p.q_weight = q_weight;
  p.k_weight = k_weight;
  p.cos_sin = cos_sin;
  p.row_index = row_index;
  p.n_rows = n_rows;
  p.ld_in = ld_in;
  p.ld_out = ld_out;
  p.rows = rows;
  p.tokens_per_sample = tokens_per_sample;
  p.d_model = d_model;
  p.head_dim = d_model / num_heads;
  p.eps = eps;
  hipStream_t s = as_stream(stream);
  const bool norm = q_weight != nullptr, rope = cos_sin != nullptr;
  int rc;
  switch (dtype) {
    case TAAC_F32: rc = dispatch_qk<float>(p, norm, rope, s, name); break;
    case TAAC_BF16: rc = dispatch_qk<bf16_t>(p, norm, rope, s, name); break;
    case TAAC_F16: rc = dispatch_qk<f16_t>(p, norm, rope, s, name); break;
    default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  }
  if (rc != TAAC_OK) return rc;
  return check_launch(name);
}

extern "C" int64_t taac_norm_bwd_workspace_floats(int64_t rows, int32_t cols, int layer_norm) {
  if (rows < 0 || cols <= 0) return -1;
  return static_cast<int64_t>(taac::kBwdMaxBlocks) * cols * (layer_norm ? 2 : 1);
}

extern "C" int taac_rmsnorm_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, float* workspace,
                                int64_t workspace_floats, int64_t rows, int32_t cols, float eps, int dtype,
                                void* stream) {
  return taac::norm_bwd_entry<false>("taac_rmsnorm_bwd", x, w, dy, dx, dw, nullptr, workspace, workspace_floats, rows,
                                     cols, eps, dtype, stream);
}

// ---- taac_rmsnorm_bwd without a caller workspace -----------------------------------------------------------------------
// The partial rows of dw live in a device array of the library image. In host code the array's name is only a handle:
// its device address is looked up once per device (every GPU holds its own copy at its own address) and that pointer
// is what the kernels receive, exactly as they receive the caller's workspace in taac_rmsnorm_bwd. Nothing has to be
// cleared between calls: a launch writes every partial row it later reads.
namespace taac {
namespace {
constexpr int64_t kStaticBwdFloats = static_cast<int64_t>(kBwdMaxBlocks) * TAAC_RMSNORM_BWD_STATIC_MAX_COLS;
static __device__ __align__(256) float scratch[kStaticBwdFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device; nullptr (with the error set) when it cannot be resolved.
float* static_scratch(const char* name) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error(TAAC_ERR_LAUNCH, "%s: cannot query the current device", name);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    float* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error(TAAC_ERR_LAUNCH, "%s: cannot resolve the device scratch array: %s", name, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}
}  // namespace
}  // namespace taac

extern "C" int taac_rmsnorm_bwd_static(const void* x, const void* w, const void* dy, void* dx, void* dw, int64_t rows,
                                       int32_t cols, float eps, int dtype, void* stream) {
  using namespace taac;
  const char* name = "taac_rmsnorm_bwd_static";
  if (cols > TAAC_RMSNORM_BWD_STATIC_MAX_COLS)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: cols=%d exceeds the %d columns the built-in scratch array covers", name,
                     cols, TAAC_RMSNORM_BWD_STATIC_MAX_COLS);
  if (rows < 0 || cols <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows must be >= 0 and cols > 0", name);
  float* ptr = static_scratch(name);
  if (ptr == nullptr) return TAAC_ERR_LAUNCH;
  return norm_bwd_entry<false>(name, x, w, dy, dx, dw, nullptr, ptr, kStaticBwdFloats, rows, cols, eps, dtype, stream);
}

extern "C" int taac_layernorm_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, void* db,
                                  float* workspace, int64_t workspace_floats, int64_t rows, int32_t cols, float eps,
                                  int dtype, void* stream) {
  return taac::norm_bwd_entry<true>("taac_layernorm_bwd", x, w, dy, dx, dw, db, workspace, workspace_floats, rows, cols,
                                    eps, dtype, stream);
}
