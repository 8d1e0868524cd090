// Backward of the SiLU-gated feed-forward (experiments/symbiosis/backbone.py:11-21, as torch autograd derives it),
// first half, as ONE token-stationary kernel for gfx950:
//
//   pre          = h W_up^T + b_up                             [M, 2F]  (recomputed in fp32, never written)
//   grad_hidden  = dy W_down                                   [M, F]   (fp32, never written)
//   hidden       = bf16( act(pre) )                            [M, F]   -> memory (operand of the down weight gradient)
//   grad_pre     = bf16( d act / d pre * grad_hidden )         [M, 2F]  -> memory (operand of the up weight gradient and
//                                                                          of the input gradient)
//
// with act(g | u) = silu(g) * u (gate first) or g * silu(u). The layer-by-layer route writes pre and grad_hidden and
// reads them back (6.3 GB at 524 288 tokens, D = 256, F = 1024); here both live in accumulator registers only.
//
// A workgroup owns 256 tokens (8 wavefronts x 32). A wavefront holds its 32 rows of h and of dy as B-operand
// fragments (2 x D/16 registers of 8 bf16) for the whole kernel. A step covers 32 hidden units: three 32 x D weight
// blocks - rows 32 s.. of the first half of W_up, of its second half, and of W_down^T - multiply h, h and dy into three
// 32 x 32 accumulators in which a lane holds, for ITS token, the same 16 hidden units of all three, so the activation
// backward is lane-local arithmetic. The weights come as a blob in fragment order (taac_swiglu_ffn_bwd_pack_weights)
// and stream L2 -> LDS by direct transfers through a ring of four 24 KB buffers, three sub-steps ahead (a sub-step is
// eight k-steps of the three blocks: half a step at D = 256, a whole one at D = 128; with two whole-step buffers, one
// step ahead, the wait for the weights was exposed in every step: 1.54 ms against the time below at 524 288 tokens);
// results leave through a wavefront-private LDS tile as 16-byte stores that cover 64-byte runs of a row.
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kFrag = 1024;                     // bytes of one 32 x 16 bf16 MFMA operand fragment
constexpr int kWaves = 8;
constexpr int kTokPerWg = kWaves * 32;
constexpr int kUnits = 32;                      // hidden units per step
constexpr int kSubK = 8;                        // k-steps (of 16 features) per sub-step
constexpr int kRing = 4;                        // weight buffers
constexpr int kTileRow = 3 * kUnits * 2 + 16;   // epilogue tile row: hidden | grad first half | grad second half | pad
constexpr int kTileWave = 32 * kTileRow;

struct FfnBwdParams {
  const bf16_t* h;        // [M, D] input of the up projection (normalised rows), row stride ldh
  const bf16_t* dy;       // [M, D] gradient of the feed-forward output, row stride lddy
  const bf16_t* packed;   // weights in fragment order
  const bf16_t* b_up;     // [2F] or null
  bf16_t* hidden;         // [M, F] row stride ldhid
  bf16_t* grad_pre;       // [M, 2F] row stride ldgp
  int64_t M, ldh, lddy, ldhid, ldgp;
  int32_t F;
};

// Blob: step s (32 hidden units), sub-step u (k-steps 8 u .. 8 u + 7) holds fragments (block b, k-step 8 u + j) at index
// b * 8 + j; block 0 = rows 32 s .. of the first half of w_up, block 1 = the same rows of its second half, block 2 =
// columns 32 s .. of w_down (rows of its transpose). Lane (l32, hh) of a fragment holds k = 16 ks + 8 hh .. + 7 of row l32.
__global__ void ffn_bwd_pack_kernel(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                    bf16x8* __restrict__ packed, int D, int F) {
  const int64_t total = static_cast<int64_t>(3) * D * F / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int NSUB = D / 16 / kSubK, NFRAG = 3 * kSubK;
  const int lane = static_cast<int>(gid % 64);
  const int f = static_cast<int>((gid / 64) % NFRAG);
  const int64_t sub = gid / 64 / NFRAG;  // step * NSUB + u
  const int64_t step = sub / NSUB;
  const int b = f / kSubK, ks = static_cast<int>(sub % NSUB) * kSubK + f % kSubK;
  const int l32 = lane % 32, hh = lane / 32;
  const int64_t unit = step * kUnits + l32;
  const int k0 = ks * 16 + hh * 8;
  bf16x8 v;
  if (b < 2) {
    v = *reinterpret_cast<const bf16x8*>(w_up + (b * static_cast<int64_t>(F) + unit) * D + k0);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = w_down[static_cast<int64_t>(k0 + e) * F + unit];
  }
  packed[gid] = v;
}

template <int N>
__device__ __forceinline__ void lds_wait_triple(bf16x8& a, bf16x8& b, bf16x8& c) {
  asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a), "+v"(b), "+v"(c) : "n"(N) : "memory");
}

template <int D, bool GATE_FIRST>
__global__ __launch_bounds__(kWaves * kWave, 2) void swiglu_ffn_bwd_hidden_kernel(const FfnBwdParams p) {
  constexpr int KS = D / 16;
  constexpr int NSUB = KS / kSubK;      // sub-steps per step
  constexpr int NFRAG = 3 * kSubK;      // fragments per sub-step
  constexpr int FPW = NFRAG / kWaves;   // transfers per wavefront and sub-step
  constexpr int kBuf = NFRAG * kFrag;
  constexpr int PRE = 3;                // fragment triples in flight
  constexpr int NST = 6;                // output stores per wavefront and step
  static_assert(KS % kSubK == 0 && NFRAG % kWaves == 0, "every wavefront stages the same number of fragments");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t* tiles = smem + kRing * kBuf;
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(tiles + kWaves * kTileWave);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int nsteps = p.F / kUnits;
  const int nsub = nsteps * NSUB;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * kTokPerWg + wave * 32;
  // Tokens at or beyond M are mapped to the last token: they compute the same values, so the duplicate stores are
  // benign and every wavefront issues the same number of memory operations (the hand-counted waits rely on that).
  auto row_of = [&](int64_t tok) -> int64_t { return tok < p.M ? tok : p.M - 1; };

  const char* w_bytes = reinterpret_cast<const char*>(p.packed);
  auto stage = [&](int q) {  // sub-step q -> ring slot q % kRing
    int ln = lane;
    asm volatile("" : "+v"(ln));
    uint8_t* base = smem + (q % kRing) * kBuf + wave * (FPW * kFrag);
    const char* src = w_bytes + (static_cast<int64_t>(q) * NFRAG + wave * FPW) * kFrag;  // scalar registers
    const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
#pragma unroll
    for (int i = 0; i < FPW; ++i) lds_dma16_offset(src + i * kFrag, lane_off, base + i * kFrag);
  };

#pragma unroll
  for (int q = 0; q < kRing - 1; ++q)
    if (q < nsub) stage(q);
  stage_bias(p.b_up, bias_lds, 2 * p.F, tid, kWaves * kWave);
  // The wavefront's 32 rows of h and of dy as B-operand fragments: lane (l32, hh) holds features 16 ks + 8 hh .. + 7 of
  // token l32. (Loading the rows contiguously and re-ordering them through LDS instead was measured: no difference.)
  bf16x8 hf[KS], df[KS];
  {
    const int64_t row = row_of(tok0 + l32);
    const bf16_t* hrow = p.h + row * p.ldh + hh * 8;
    const bf16_t* drow = p.dy + row * p.lddy + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) hf[ks] = *reinterpret_cast<const bf16x8*>(hrow + ks * 16);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) df[ks] = *reinterpret_cast<const bf16x8*>(drow + ks * 16);
    // consumed here, so that the compiler's wait for the rows sits in front of the loop and not inside it
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(hf[ks]), "+v"(df[ks]));
  }
  // memory rows of the epilogue stores: piece i = token 16 * i + lane / 4
  int64_t prow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) prow[i] = row_of(tok0 + i * 16 + lane / 4);
  vm_wait<0>();
  __syncthreads();

  uint8_t* tile = tiles + wave * kTileWave;
  for (int s = 0; s < nsteps; ++s) {
    // the up-projection accumulators start from the bias (accumulator order: register jq * 4 + e of lane (l32, hh) is
    // hidden unit 32 s + jq * 8 + hh * 4 + e of token l32)
    f32x16 acc_a, acc_b, acc_d;
    {
      const bf16_t* bias = bias_lds + s * kUnits + hh * 4;
#pragma unroll
      for (int jq = 0; jq < 4; ++jq) {
        const bf16x4 ba = *reinterpret_cast<const bf16x4*>(bias + jq * 8);
        const bf16x4 bb = *reinterpret_cast<const bf16x4*>(bias + p.F + jq * 8);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc_a[jq * 4 + e] = static_cast<float>(ba[e]);
          acc_b[jq * 4 + e] = static_cast<float>(bb[e]);
          acc_d[jq * 4 + e] = 0.f;
        }
      }
    }
    static_for<NSUB>([&](auto u) {
      constexpr int U = decltype(u)::value;
      const int q = s * NSUB + U;
      // slot (q + 3) % 4 was last read in sub-step q - 1, which every wavefront has left
      if (q + kRing - 1 < nsub) stage(q + kRing - 1);
      const uint32_t wb = lds_offset(smem) + (q % kRing) * kBuf + lane * 16;
      bf16x8 fa[PRE], fb[PRE], fd[PRE];
      static_for<PRE>([&](auto k) {
        constexpr int K_ = decltype(k)::value;
        lds_read_frag<K_ * kFrag>(fa[K_], wb);
        lds_read_frag<(kSubK + K_) * kFrag>(fb[K_], wb);
        lds_read_frag<(2 * kSubK + K_) * kFrag>(fd[K_], wb);
      });
      static_for<kSubK>([&](auto k) {
        constexpr int K_ = decltype(k)::value;
        constexpr int R = K_ % PRE;
        // reads issued behind triple K_: the triples up to min(K_ + PRE - 1, kSubK - 1)
        constexpr int newest = K_ + PRE - 1 < kSubK - 1 ? K_ + PRE - 1 : kSubK - 1;
        lds_wait_triple<3 * (newest - K_)>(fa[R], fb[R], fd[R]);
        acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[R], hf[U * kSubK + K_], acc_a, 0, 0, 0);
        acc_b = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[R], hf[U * kSubK + K_], acc_b, 0, 0, 0);
        acc_d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fd[R], df[U * kSubK + K_], acc_d, 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (K_ + PRE < kSubK) {
          lds_read_frag<(K_ + PRE) * kFrag>(fa[R], wb);
          lds_read_frag<(kSubK + K_ + PRE) * kFrag>(fb[R], wb);
          lds_read_frag<(2 * kSubK + K_ + PRE) * kFrag>(fd[R], wb);
        }
      });
      if constexpr (U == NSUB - 1) {
        // ---- activation backward, lane-local and in fp32 (the up projection and dy w_down are not rounded on the way,
        //      as in the fused forward kernel) ---------------------------------------------------------------------------------
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          bf16x4 hv, ga, gb;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a = acc_a[jq * 4 + e], b = acc_b[jq * 4 + e], d = acc_d[jq * 4 + e];
            const float act = GATE_FIRST ? a : b;  // the operand that goes through SiLU
            const float lin = GATE_FIRST ? b : a;  // the one that multiplies it
            const float sig = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * act));
            const float silu = act * sig;
            const float dact = (d * lin) * fmaf(silu, 1.f - sig, sig);  // silu'(x) = sig + silu * (1 - sig)
            const float dlin = d * silu;
            hv[e] = static_cast<bf16_t>(silu * lin);
            ga[e] = static_cast<bf16_t>(GATE_FIRST ? dact : dlin);
            gb[e] = static_cast<bf16_t>(GATE_FIRST ? dlin : dact);
          }
          uint8_t* dst = tile + l32 * kTileRow + (jq * 8 + hh * 4) * 2;
          *reinterpret_cast<bf16x4*>(dst) = hv;
          *reinterpret_cast<bf16x4*>(dst + kUnits * 2) = ga;
          *reinterpret_cast<bf16x4*>(dst + 2 * kUnits * 2) = gb;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // ---- row-wise out of the tile: lane -> token 16 * i + lane / 4, 16-byte piece lane % 4 of each 64-byte run --------
        const int unit0 = s * kUnits + (lane % 4) * 8;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const uint8_t* src = tile + (i * 16 + lane / 4) * kTileRow + (lane % 4) * 16;
          const bf16x8 hv = *reinterpret_cast<const bf16x8*>(src);
          const bf16x8 ga = *reinterpret_cast<const bf16x8*>(src + kUnits * 2);
          const bf16x8 gb = *reinterpret_cast<const bf16x8*>(src + 2 * kUnits * 2);
          // streaming stores: 6 KB per token leave the kernel and nothing of it is read again here (1.50 -> 1.34 ms)
          __builtin_nontemporal_store(hv, reinterpret_cast<bf16x8*>(p.hidden + prow[i] * p.ldhid + unit0));
          __builtin_nontemporal_store(ga, reinterpret_cast<bf16x8*>(p.grad_pre + prow[i] * p.ldgp + unit0));
          __builtin_nontemporal_store(gb, reinterpret_cast<bf16x8*>(p.grad_pre + prow[i] * p.ldgp + p.F + unit0));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
      if (q + 1 < nsub) {
        // The transfers of sub-step q + 1 were issued at the start of sub-step q - 2 (or in front of the loop, where
        // everything was awaited). Behind them this wavefront has issued at least: the transfers of q + 2 and q + 3 (where
        // those exist) and the stores of the epilogues in sub-steps q - 1 and q (one of the two at D = 256, both at D = 128).
        constexpr int kStores = NST * (NSUB == 1 ? 2 : 1);
        if (q + 3 < nsub) vm_wait<kStores + 2 * FPW>();
        else if (q + 2 < nsub) vm_wait<kStores + FPW>();
        else vm_wait<kStores>();
        __syncthreads();
      }
    });
  }
}

size_t bwd_lds_bytes(int32_t D, int32_t F) {
  return static_cast<size_t>(kRing) * 3 * kSubK * kFrag + kWaves * kTileWave + static_cast<size_t>(2) * F * 2;
}

bool bwd_shape_ok(int32_t D, int32_t F) {
  return (D == 128 || D == 256) && F > 0 && F % kUnits == 0 && bwd_lds_bytes(D, F) <= 160 * 1024;
}

template <int D>
int launch_bwd_hidden(const FfnBwdParams& p, bool gate_first, hipStream_t s, const char* name) {
  const size_t lds_bytes = bwd_lds_bytes(D, p.F);
  const int64_t grid = (p.M + kTokPerWg - 1) / kTokPerWg;
  if (grid > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  auto go = [&](auto kernel) -> int {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds_bytes)) != hipSuccess)
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);
    hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(kWaves * kWave), lds_bytes, s, p);
    return check_launch(name);
  };
  return gate_first ? go(swiglu_ffn_bwd_hidden_kernel<D, true>) : go(swiglu_ffn_bwd_hidden_kernel<D, false>);
}


}  // namespace
}  // namespace taac

extern "C" int64_t taac_swiglu_ffn_bwd_packed_bytes(int32_t D, int32_t F) {
  if (!taac::bwd_shape_ok(D, F)) return -1;
  return static_cast<int64_t>(3) * D * F * 2;
}

extern "C" int taac_swiglu_ffn_bwd_pack_weights(const void* w_up, const void* w_down, void* packed, int32_t D, int32_t F,
                                                void* stream) {
  using namespace taac;
  const char* name = "taac_swiglu_ffn_bwd_pack_weights";
  if (!bwd_shape_ok(D, F))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: built for D = 128 / 256 and F a multiple of 32 up to about 2048 (got D=%d, F=%d)", name, D, F);
  if (!w_up || !w_down || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!aligned16(w_up) || !aligned16(packed))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: w_up and packed must be 16-byte aligned", name);
  const int64_t total = static_cast<int64_t>(3) * D * F / 8;
  hipLaunchKernelGGL(ffn_bwd_pack_kernel, dim3(static_cast<uint32_t>((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const bf16_t*>(w_up), static_cast<const bf16_t*>(w_down), static_cast<bf16x8*>(packed), D, F);
  return check_launch(name);
}

extern "C" int taac_swiglu_ffn_bwd_hidden(const void* h, int64_t ldh, const void* dy, int64_t lddy, const void* packed,
                                          const void* b_up, void* hidden, int64_t ldhid, void* grad_pre, int64_t ldgp,
                                          int64_t M, int32_t D, int32_t F, int gate_first, void* stream) {
  using namespace taac;
  const char* name = "taac_swiglu_ffn_bwd_hidden";
  if (M < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0", name);
  if (!bwd_shape_ok(D, F))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: built for D = 128 / 256 and F a multiple of 32 up to about 2048 (got D=%d, F=%d)", name, D, F);
  if (ldh % 8 != 0 || lddy % 8 != 0 || ldhid % 8 != 0 || ldgp % 8 != 0 || ldh < D || lddy < D || ldhid < F || ldgp < 2 * F)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: row strides must be multiples of 8 and cover a row", name);
  if (M == 0) return TAAC_OK;
  if (!h || !dy || !packed || !hidden || !grad_pre) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!aligned16(h) || !aligned16(dy) || !aligned16(packed) || !aligned16(hidden) || !aligned16(grad_pre) ||
      (b_up && !aligned16(b_up)))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  FfnBwdParams p;
  p.h = static_cast<const bf16_t*>(h);
  p.dy = static_cast<const bf16_t*>(dy);
  p.packed = static_cast<const bf16_t*>(packed);
  p.b_up = static_cast<const bf16_t*>(b_up);
  p.hidden = static_cast<bf16_t*>(hidden);
  p.grad_pre = static_cast<bf16_t*>(grad_pre);
  p.M = M;
  p.ldh = ldh;
  p.lddy = lddy;
  p.ldhid = ldhid;
  p.ldgp = ldgp;
  p.F = F;
  hipStream_t s = as_stream(stream);
  return D == 256 ? launch_bwd_hidden<256>(p, gate_first != 0, s, name) : launch_bwd_hidden<128>(p, gate_first != 0, s, name);
}
