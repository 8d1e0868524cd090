// Readout of the unified token backbone for gfx950, one kernel per batch:
//   tokens -> [RMSNorm per token] -> concat( token[cls], token[candidate] or 0, masked mean over the valid tokens )
//          -> [RMSNorm over the 3D features] -> [Linear(3D, hidden) -> SiLU -> Linear(hidden, actions) [-> sigmoid]]
// Replaces final_norm + CandidateClsPooler.forward + the classifier of PCVRSymbiosis (experiments/symbiosis/
// model.py:215-222, 291, 309, 316-317; experiments/symbiosis/pooling.py:16-32) and masked_mean
// (modeling/sequence.py:54-60) without writing the normalised tokens, the pooled vector or the hidden layer to memory.
//
// One workgroup of 256 lanes per sample. The sample's valid token rows are read exactly once: a row is owned by 32
// consecutive lanes (128-bit loads, up to four per lane), 16 to 32 rows in flight per workgroup; the token norm's
// statistic is a 32-lane shuffle reduction, the normalised row is accumulated in fp32 registers. Because the token
// norm's weight is per feature it commutes with the mean and is applied once to the pooled sum. The classifier is two
// matrix-vector products against weights that stay in L2: a weight row is read by 32 lanes as contiguous 16-byte
// pieces, the pooled vector and the hidden layer live in LDS as fp32. Everything is evaluated in fp32 from the stored
// bf16 operands and rounded once where a bf16 result is written.

#include "common.h"

namespace taac {
namespace {

constexpr int kRowLanes = 32;                           // lanes that own one token row
constexpr int kMaxWidth = 1024;                         // model width and classifier hidden size limit

struct ReadoutParams {
  const bf16_t* tokens;         // [B, T, D]
  const int32_t* key_lengths;   // [B] or null
  const uint32_t* valid_bits;   // [B, ceil(T / 32)] or null
  int32_t T, D;
  int32_t cls_index, candidate_index;  // candidate_index < 0: that third of the pooled vector is zero
  const bf16_t* token_norm_w;   // [D] or null (tokens are used as they are)
  const bf16_t* pool_norm_w;    // [3D] or null
  float eps;
  const bf16_t* fc1_w;          // [hidden, 3D] or null (no classifier)
  const bf16_t* fc1_b;          // [hidden] or null
  const bf16_t* fc2_w;          // [actions, hidden]
  const bf16_t* fc2_b;          // [actions] or null
  int32_t hidden, actions;
  bf16_t* embedding_out;        // [B, 3D] or null
  float* logits_out;            // [B, actions] or null
  int32_t apply_sigmoid;
};

// Loads the NV 16-byte pieces of a row that this lane owns (piece l32 + 32 * i) and returns its part of the row's sum
// of squares.
template <int NV>
__device__ __forceinline__ float load_row(const bf16_t* row, int nvec, int l32, bf16x8 (&v)[NV]) {
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int piece = l32 + kRowLanes * i;
    if (piece < nvec) {
      v[i] = *reinterpret_cast<const bf16x8*>(row + piece * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = static_cast<float>(v[i][e]);
        ss = fmaf(f, f, ss);
      }
    }
  }
  return ss;
}

template <int NV, int kReadoutBlock>
__global__ __launch_bounds__(kReadoutBlock) void candidate_readout_kernel(const ReadoutParams p) {
  constexpr int kRowGroups = kReadoutBlock / kRowLanes;  // lane groups, each owning one token row at a time
  // LDS: [pooled: 3D floats = cls | candidate | mean, later the normalised embedding]
  //      [partial sums of the mean, kRowGroups x D floats; later the hidden layer]
  extern __shared__ __attribute__((aligned(16))) float s_dyn[];
  __shared__ float s_scalar[kRowGroups];
  __shared__ int s_count[kRowGroups];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int g = tid / kRowLanes;
  const int l32 = tid % kRowLanes;
  const int D = p.D, T = p.T;
  float* s_pooled = s_dyn;
  float* s_red = s_dyn + 3 * D;  // row i of the partial sums starts at s_red + i * D
  const int nvec = D / 8;
  const bf16_t* xb = p.tokens + static_cast<int64_t>(b) * T * D;
  const int wpr = (T + 31) / 32;
  int t_end = T;
  if (p.key_lengths != nullptr) {
    const int len = p.key_lengths[b];
    t_end = len < 0 ? 0 : (len > T ? T : len);
  }

  // ---- masked mean of the (normalised) tokens: kRows rows per group in flight ----------------------------------------
  constexpr int kRows = NV <= 2 ? 4 : 2;
  float acc[NV][8];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;
  int count = 0;
  for (int t0 = g; t0 < t_end; t0 += kRowGroups * kRows) {
    bf16x8 v[kRows][NV];
    float ss[kRows];
    bool ok[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int t = t0 + r * kRowGroups;
      ok[r] = t < t_end;
      if (ok[r] && p.valid_bits != nullptr)
        ok[r] = ((p.valid_bits[static_cast<int64_t>(b) * wpr + t / 32] >> (t % 32)) & 1u) != 0u;
      ss[r] = 0.f;
      if (ok[r]) ss[r] = load_row<NV>(xb + static_cast<int64_t>(t) * D, nvec, l32, v[r]);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (!ok[r]) continue;  // uniform over the 32 lanes of the group
      float scale = 1.0f;
      if (p.token_norm_w != nullptr) scale = rsqrtf(group_sum<kRowLanes>(ss[r]) * (1.0f / D) + p.eps);
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (l32 + kRowLanes * i < nvec) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[i][e] = fmaf(static_cast<float>(v[r][i][e]), scale, acc[i][e]);
        }
      ++count;
    }
  }
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if (l32 + kRowLanes * i < nvec) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s_red[g * D + (l32 + kRowLanes * i) * 8 + e] = acc[i][e];
    }
  if (l32 == 0) s_count[g] = count;

  // ---- the two picked tokens: group 0 the cls token, group 1 the candidate token -------------------------------------
  if (g < 2) {
    const int index = g == 0 ? p.cls_index : p.candidate_index;
    bf16x8 v[NV];
    float scale = 0.f;  // a missing candidate contributes zeros
    if (index >= 0) {
      const float ss = load_row<NV>(xb + static_cast<int64_t>(index) * D, nvec, l32, v);
      scale = p.token_norm_w != nullptr ? rsqrtf(group_sum<kRowLanes>(ss) * (1.0f / D) + p.eps) : 1.0f;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int piece = l32 + kRowLanes * i;
      if (piece < nvec) {
        bf16x8 w;
        if (p.token_norm_w != nullptr) w = *reinterpret_cast<const bf16x8*>(p.token_norm_w + piece * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float x = index >= 0 ? static_cast<float>(v[i][e]) * scale : 0.f;
          s_pooled[g * D + piece * 8 + e] = p.token_norm_w != nullptr ? x * static_cast<float>(w[e]) : x;
        }
      }
    }
  }
  __syncthreads();
  int valid = 0;
#pragma unroll
  for (int i = 0; i < kRowGroups; ++i) valid += s_count[i];
  const float inv_count = 1.0f / static_cast<float>(valid < 1 ? 1 : valid);
  for (int f = tid; f < D; f += kReadoutBlock) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kRowGroups; ++i) s += s_red[i * D + f];
    s *= inv_count;
    s_pooled[2 * D + f] = p.token_norm_w != nullptr ? s * static_cast<float>(p.token_norm_w[f]) : s;
  }
  __syncthreads();

  // ---- RMSNorm over the 3D pooled features ---------------------------------------------------------------------------
  const int K = 3 * D;
  if (p.pool_norm_w != nullptr) {
    float ss = 0.f;
    for (int f = tid; f < K; f += kReadoutBlock) ss = fmaf(s_pooled[f], s_pooled[f], ss);
    ss = group_sum<kRowLanes>(ss);
    if (l32 == 0) s_scalar[g] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < kRowGroups; ++i) total += s_scalar[i];
    const float scale = rsqrtf(total * (1.0f / K) + p.eps);
    for (int f = tid; f < K; f += kReadoutBlock) s_pooled[f] = s_pooled[f] * scale * static_cast<float>(p.pool_norm_w[f]);
    __syncthreads();
  }
  if (p.embedding_out != nullptr) {
    bf16_t* dst = p.embedding_out + static_cast<int64_t>(b) * K;
    for (int f = tid; f < K; f += kReadoutBlock) dst[f] = static_cast<bf16_t>(s_pooled[f]);
  }
  if (p.fc1_w == nullptr) return;

  // ---- classifier: hidden = silu(W1 e + b1), logits = W2 hidden + b2 ------------------------------------------------
  float* s_hidden = s_red;  // the partial sums are dead (barriers above); the host sizes the region for both uses
  const int kvec = K / 8;
  for (int j = g; j < p.hidden; j += kRowGroups) {
    const bf16_t* wrow = p.fc1_w + static_cast<int64_t>(j) * K;
    float dot = 0.f;
    for (int piece = l32; piece < kvec; piece += kRowLanes) {
      const bf16x8 w = *reinterpret_cast<const bf16x8*>(wrow + piece * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf(static_cast<float>(w[e]), s_pooled[piece * 8 + e], dot);
    }
    dot = group_sum<kRowLanes>(dot);
    if (l32 == 0) {
      const float z = dot + (p.fc1_b != nullptr ? static_cast<float>(p.fc1_b[j]) : 0.f);
      s_hidden[j] = z / (1.0f + expf(-z));
    }
  }
  __syncthreads();
  for (int a = g; a < p.actions; a += kRowGroups) {
    const bf16_t* wrow = p.fc2_w + static_cast<int64_t>(a) * p.hidden;
    float dot = 0.f;
    for (int j = l32; j < p.hidden; j += kRowLanes) dot = fmaf(static_cast<float>(wrow[j]), s_hidden[j], dot);
    dot = group_sum<kRowLanes>(dot);
    if (l32 == 0) {
      float z = dot + (p.fc2_b != nullptr ? static_cast<float>(p.fc2_b[a]) : 0.f);
      if (p.apply_sigmoid) z = 1.0f / (1.0f + expf(-z));
      p.logits_out[static_cast<int64_t>(b) * p.actions + a] = z;
    }
  }
}

}  // namespace
}  // namespace taac

extern "C" int taac_candidate_readout_fwd(const void* tokens, const int32_t* key_lengths, const uint32_t* valid_bits,
                                          int32_t B, int32_t T, int32_t D, int32_t cls_index, int32_t candidate_index,
                                          const void* token_norm_weight, const void* pool_norm_weight, float eps,
                                          const void* fc1_weight, const void* fc1_bias, int32_t hidden,
                                          const void* fc2_weight, const void* fc2_bias, int32_t actions,
                                          void* embedding_out, float* logits_out, int apply_sigmoid, void* stream) {
  using namespace taac;
  const char* name = "taac_candidate_readout_fwd";
  if (B < 0 || T <= 0 || D <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: B >= 0 and T, D > 0 required", name);
  if (D % 8 != 0 || D > kMaxWidth)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D=%d must be a multiple of 8 and at most %d", name, D, kMaxWidth);
  if (cls_index < 0 || cls_index >= T || candidate_index >= T)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: token index outside the sequence", name);
  if (key_lengths != nullptr && valid_bits != nullptr)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: give key_lengths or valid_bits, not both", name);
  const bool classifier = fc1_weight != nullptr;
  if (classifier) {
    if (hidden <= 0 || actions <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: hidden and actions must be positive", name);
    if (hidden > kMaxWidth) return set_error(TAAC_ERR_UNSUPPORTED, "%s: hidden=%d above %d", name, hidden, kMaxWidth);
    if (!fc2_weight || !logits_out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: the classifier needs fc2_weight and logits_out", name);
  } else if (!embedding_out) {
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: nothing to compute: no classifier and no embedding_out", name);
  }
  if (B == 0) return TAAC_OK;
  if (!tokens) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!aligned16(tokens) || !aligned16(token_norm_weight) || !aligned16(fc1_weight))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tokens, token_norm_weight and fc1_weight must be 16-byte aligned", name);
  ReadoutParams p{};
  p.tokens = static_cast<const bf16_t*>(tokens);
  p.key_lengths = key_lengths;
  p.valid_bits = valid_bits;
  p.T = T;
  p.D = D;
  p.cls_index = cls_index;
  p.candidate_index = candidate_index;
  p.token_norm_w = static_cast<const bf16_t*>(token_norm_weight);
  p.pool_norm_w = static_cast<const bf16_t*>(pool_norm_weight);
  p.eps = eps;
  p.fc1_w = static_cast<const bf16_t*>(fc1_weight);
  p.fc1_b = static_cast<const bf16_t*>(fc1_bias);
  p.fc2_w = static_cast<const bf16_t*>(fc2_weight);
  p.fc2_b = static_cast<const bf16_t*>(fc2_bias);
  p.hidden = classifier ? hidden : 0;
  p.actions = classifier ? actions : 0;
  p.embedding_out = static_cast<bf16_t*>(embedding_out);
  p.logits_out = logits_out;
  p.apply_sigmoid = apply_sigmoid ? 1 : 0;
  hipStream_t s = as_stream(stream);
  const int nv = (D / 8 + kRowLanes - 1) / kRowLanes;
  // Long sequences get 1024-lane workgroups: a sample's rows are spread over 32 lane groups, and because only two such
  // workgroups fit a compute unit at a time the rest are handed out as others finish, which evens out samples of very
  // different lengths. Short sequences keep 256 lanes (more workgroups per compute unit, cheaper reduction).
  const bool wide = T >= 128;
  const int threads = wide ? 1024 : 256;
  const int groups = threads / kRowLanes;
  const int region = groups * D > p.hidden ? groups * D : p.hidden;
  const size_t lds = static_cast<size_t>(3 * D + region) * sizeof(float);  // at most 140 KB
  const dim3 grid(static_cast<uint32_t>(B)), block(threads);
#define TAAC_READOUT_LAUNCH(NV)                                                                                        \
  do {                                                                                                                 \
    auto kernel = wide ? candidate_readout_kernel<NV, 1024> : candidate_readout_kernel<NV, 256>;                       \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,         \
                            static_cast<int>(lds)) != hipSuccess)                                                      \
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds);                             \
    hipLaunchKernelGGL(kernel, grid, block, lds, s, p);                                                                \
  } while (0)
  switch (nv) {
    case 1: TAAC_READOUT_LAUNCH(1); break;
    case 2: TAAC_READOUT_LAUNCH(2); break;
    case 3: TAAC_READOUT_LAUNCH(3); break;
    default: TAAC_READOUT_LAUNCH(4); break;
  }
#undef TAAC_READOUT_LAUNCH
  return check_launch(name);
}
