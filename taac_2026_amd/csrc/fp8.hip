// Per-tensor FP8 (OCP e4m3fn) scaling helpers for gfx950: absolute maximum and quantisation.
// scale = max(amax, tiny) / 448; q = round_to_nearest_even(clamp(x / scale, +-448)).
#include "common.h"

namespace taac {
namespace {

constexpr int kBlock = 256;

__global__ void amax_clear_kernel(float* out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *out = 0.f;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void amax_kernel(const T* __restrict__ x, int64_t n, float* out) {
  __shared__ float s_part[kBlock / kWave];
  float m = 0.f;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  constexpr int VEC = 16 / sizeof(T);
  const int64_t nvec = aligned16(x) ? n / VEC : 0;
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  const vec_t* xv = reinterpret_cast<const vec_t*>(x);
  // Four independent 16-byte loads per thread and trip keep enough bytes in flight to stream from HBM.
  int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  for (; i + 3 * stride < nvec; i += 4 * stride) {
    vec_t v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(xv + i + u * stride);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < VEC; ++e) m = fmaxf(m, fabsf(static_cast<float>(v[u][e])));
  }
  for (; i < nvec; i += stride) {
    const vec_t v = xv[i];
#pragma unroll
    for (int e = 0; e < VEC; ++e) m = fmaxf(m, fabsf(static_cast<float>(v[e])));
  }
  for (int64_t i = nvec * VEC + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
    m = fmaxf(m, fabsf(static_cast<float>(x[i])));
  m = group_max<kWave>(m);
  if (threadIdx.x % kWave == 0) s_part[threadIdx.x / kWave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kBlock / kWave; ++w) m = fmaxf(m, s_part[w]);
    // Non-negative floats order like their bit patterns; NaN inputs are ignored by fmaxf.
    atomicMax(reinterpret_cast<unsigned int*>(out), __float_as_uint(m));
  }
}

__device__ __forceinline__ uint8_t to_e4m3(float v) {
  v = __builtin_fminf(__builtin_fmaxf(v, -448.f), 448.f);
  const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false);
  return static_cast<uint8_t>(packed & 0xff);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void quantize_fp8_kernel(const T* __restrict__ x, int64_t n,
                                                              const float* __restrict__ amax, uint8_t* __restrict__ q) {
  const float scale = fmaxf(*amax, 1e-12f) / 448.0f;
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * 8;
  if (base >= n) return;
  if (base + 8 <= n && ((reinterpret_cast<uintptr_t>(q) & 7u) == 0)) {
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
      f[e] = __builtin_fminf(__builtin_fmaxf(static_cast<float>(x[base + e]) / scale, -448.f), 448.f);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
    u32x2 r = {static_cast<uint32_t>(lo), static_cast<uint32_t>(hi)};
    *reinterpret_cast<u32x2*>(q + base) = r;
  } else {
    for (int64_t i = base; i < n && i < base + 8; ++i) q[i] = to_e4m3(static_cast<float>(x[i]) / scale);
  }
}

}  // namespace
}  // namespace taac

extern "C" int taac_amax(const void* x, int64_t n, int dtype, float* amax_out, void* stream) {
  using namespace taac;
  const char* name = "taac_amax";
  if (n < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: n must be >= 0", name);
  if (!amax_out || (n > 0 && !x)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(amax_clear_kernel, dim3(1), dim3(kWave), 0, s, amax_out);
  if (n > 0) {
    int64_t blocks = (n / 8 + kBlock - 1) / kBlock;
    if (blocks < 1) blocks = 1;
    if (blocks > 256 * 16) blocks = 256 * 16;
    switch (dtype) {
      case TAAC_F32:
        hipLaunchKernelGGL((amax_kernel<float>), dim3(blocks), dim3(kBlock), 0, s, static_cast<const float*>(x), n,
                           amax_out);
        break;
      case TAAC_BF16:
        hipLaunchKernelGGL((amax_kernel<bf16_t>), dim3(blocks), dim3(kBlock), 0, s, static_cast<const bf16_t*>(x), n,
                           amax_out);
        break;
      case TAAC_F16:
        hipLaunchKernelGGL((amax_kernel<f16_t>), dim3(blocks), dim3(kBlock), 0, s, static_cast<const f16_t*>(x), n,
                           amax_out);
        break;
      default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
    }
  }
  return check_launch(name);
}

extern "C" int taac_quantize_fp8(const void* x, int64_t n, int dtype, const float* amax, void* q, void* stream) {
  using namespace taac;
  const char* name = "taac_quantize_fp8";
  if (n < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: n must be >= 0", name);
  if (n == 0) return TAAC_OK;
  if (!x || !amax || !q) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  hipStream_t s = as_stream(stream);
  const int64_t blocks = ((n + 7) / 8 + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor too large", name);
  uint8_t* qq = static_cast<uint8_t*>(q);
  switch (dtype) {
    case TAAC_F32:
      hipLaunchKernelGGL((quantize_fp8_kernel<float>), dim3(blocks), dim3(kBlock), 0, s, static_cast<const float*>(x),
                         n, amax, qq);
      break;
    case TAAC_BF16:
      hipLaunchKernelGGL((quantize_fp8_kernel<bf16_t>), dim3(blocks), dim3(kBlock), 0, s,
                         static_cast<const bf16_t*>(x), n, amax, qq);
      break;
    case TAAC_F16:
      hipLaunchKernelGGL((quantize_fp8_kernel<f16_t>), dim3(blocks), dim3(kBlock), 0, s, static_cast<const f16_t*>(x),
                         n, amax, qq);
      break;
    default: return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown dtype %d", name, dtype);
  }
  return check_launch(name);
}
