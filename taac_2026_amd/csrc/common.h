// Shared device/host helpers for the gfx950 kernels of libtaac_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/taac_hip.h"

namespace taac {

// ---- vector / element types -------------------------------------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;
typedef __attribute__((__vector_size__(8 * sizeof(int)))) int i32x8;

constexpr int kWave = 64;     // CDNA wavefront width
constexpr int kNumXcd = 8;    // MI355X: 8 accelerator dies, workgroup i is dispatched to die i % 8

// ---- host-side error plumbing -----------------------------------------------------------------------------------
int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);
// Compute units of the current device, cached per device; -1 when the query fails.
int compute_units();
// Values set through taac_test_hooks: a cap on the grid of the persistent kernels (0: none) and whether taac_linear_fp8
// is routed to its tiled kernel.
int test_max_workgroups();
bool test_fp8_tiled();
// Packs the qkv / out / feed-forward weights (gate first) of n backbone blocks into fragment order (ffn.hip).
// fold_act: the up projection also takes the constants of the gate's activation (the kernels are then called with
// TAAC_FOLDED_ACTIVATION; allowed where ffn_act_fold_supported says so).
int pack_backbone_blocks(const taac_block_weights* blocks, int n, int32_t D, int32_t F, void* const* packed_qkv,
                         void* const* packed_out, void* const* packed_ffn, bool fold_act, hipStream_t s, const char* name);
bool ffn_act_fold_supported(int32_t D, int32_t F);
// RMSNorm + q | k | v projection with the query / key epilogue (ffn.hip; the arguments of taac_norm_linear_qk_fwd with
// packed weights) whose output is a stack of per-head planes [3 * num_heads][M][head_dim], head_dim 32 or 64.
int norm_linear_qk_heads(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* bias,
                         const void* packed_weights, void* out, int64_t M, int32_t d_model, int32_t num_heads,
                         int32_t tokens_per_sample, const void* qk_weight, const void* cos_sin, float* qk_sumsq,
                         const int32_t* rows, const int32_t* n_rows, int norm_folded, void* stream);
// Out projection + feed-forward half of a block (ffn.hip; attn_plane: 0 = rows of ld_attn elements, 32 / 64 = per-head
// planes) that also writes the dot product of every stored output row with head_w to token_dots[row].
int attn_out_ffn_readout(const void* attn, int64_t ld_attn, int attn_plane, const void* out_bias,
                         const void* packed_out_weights, const void* residual, int64_t ldr, const void* norm_weight,
                         float eps, const void* b_up, const void* b_down, const void* packed_ffn_weights, void* out,
                         int64_t ldo, int64_t M, int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows,
                         int norm_folded, const void* head_w, float* token_dots, void* stream);
// Token-stationary e4m3 dense layer (fp8_ts.hip): TAAC_OK after a launch, a negative status on an error, 1 when the shape
// is not covered and the caller must use the tiled kernel.
int launch_linear_fp8_ts(const void* a, int a_is_fp8, int64_t lda, const void* w, const float* amax_a,
                         const float* amax_w, const void* bias, const void* residual, void* out, int64_t ldo,
                         int64_t M, int32_t N, int32_t K, int epilogue, int gate_first, hipStream_t s,
                         const char* name);

// FP8 preparation of a backbone (ffn_fp8.hip): per block four weight scales (qkv, out, up, down; zeroed by the caller), the row-major e4m3
// copies of the qkv / out weights and the packed feed-forward blob.
int prepare_backbone_fp8(const taac_block_weights* blocks, int n, int32_t D, int32_t F, float* const* scales,
                         void* const* qkv_q, void* const* out_q, void* const* ffn_blob, hipStream_t s, const char* name);
// p[0..n) = 0 with a kernel (ffn_fp8.hip).
int fill_zero(float* p, int n, hipStream_t s, const char* name);
// *out (zeroed by the caller) = max over the (listed) rows of | bf16(rmsnorm(x, w, eps)) |, rows of 256 bf16 features
// (ffn_fp8.hip).
int rmsnorm_amax_256(const void* x, int64_t ldx, const void* w, float eps, int64_t M, const int32_t* rows,
                     const int32_t* n_rows, float* out, hipStream_t s, const char* name);

// Set (per host thread) while taac_backbone_fwd drives the FP8 entry points: it has zeroed every maximum of the forward in
// one launch, so the entry points skip the clearing launch each of them issues for its own outputs.
inline thread_local bool maxima_precleared = false;
struct PreclearedMaxima {
  PreclearedMaxima() { maxima_precleared = true; }
  ~PreclearedMaxima() { maxima_precleared = false; }
};

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
__host__ __device__ inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device helpers ---------------------------------------------------------------------------------------------
template <typename T>
struct Vec8;  // eight 16-bit elements = one 128-bit access
template <>
struct Vec8<bf16_t> {
  typedef bf16x8 type;
  typedef bf16x4 half_type;
};
template <>
struct Vec8<f16_t> {
  typedef f16x8 type;
  typedef f16x4 half_type;
};

__device__ __forceinline__ float wave_shfl_xor(float v, int mask) { return __shfl_xor(v, mask, kWave); }

// Sum / max over groups of G consecutive lanes (G a power of two <= 64). Every lane of a group gets the result.
template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Logical -> physical workgroup id so that consecutive logical ids run on the same accelerator die (and share its
// L2). Hardware sends physical id p to die p % 8; die x is given the contiguous logical range starting at
// x * (total / 8) + min(x, total % 8).
__device__ __forceinline__ uint32_t xcd_remap(uint32_t pid, uint32_t total) {
  const uint32_t xcd = pid % kNumXcd;
  const uint32_t local = pid / kNumXcd;
  const uint32_t base = total / kNumXcd;
  const uint32_t rem = total % kNumXcd;
  const uint32_t start = xcd * base + (xcd < rem ? xcd : rem);
  return start + local;
}

}  // namespace taac
