// MoE router for gfx950: softmax over experts, top-k selection, optional renormalisation.
//
// Semantics follow the router the reference's fused_moe is fed with
// (python/dlBLAS/tests/kernels/test_fused_moe.py:213-216: softmax in fp32, then top-k;
// python/dlBLAS/dlblas/kernels/fused_moe.py:322-323: weights / weights.sum(-1)), with the two
// points the reference leaves open fixed here: selection runs on the logits (the softmax is
// monotone, so this is the same order without depending on exp rounding) and equal logits
// resolve to the lowest expert index.  The fused softmax + K x argmax structure is that of
// python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:24-60; indices are written directly, and
// that kernel's own outputs (the full softmax and the [K, S, E] int64 one-hot masks) on request.
//
// Mapping: a token is owned by one DPP row (16 lanes); every lane holds VPL consecutive
// experts (VPL = 4 covers E <= 64 with one 128-bit load per lane), so a wave processes four
// tokens and every reduction (max, sum, K argmax rounds) is four DPP steps with no LDS.
#include "common.h"

namespace dlb {
namespace {

// order-preserving map float -> uint32 (larger float <=> larger key); -0.0 < +0.0 there, so
// canonicalise zeros first to keep "equal logits -> lowest index".
__device__ __forceinline__ uint32_t orderable(float f) {
  f = (f == 0.0f) ? 0.0f : f;
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// max of (key, tag) pairs over a DPP row, lexicographic on (key, tag).
template <int CTRL>
__device__ __forceinline__ void row_step_max(uint32_t& key, uint32_t& tag) {
  const uint32_t ok = dpp_u32<CTRL>(key);
  const uint32_t ot = dpp_u32<CTRL>(tag);
  const bool take = (ok > key) || (ok == key && ot > tag);
  key = take ? ok : key;
  tag = take ? ot : tag;
}

// The logits of one token, VPL consecutive experts per lane of its DPP row (-inf past E and for
// dead rows).  LT = element type of the logits (fp32, or bf16 / fp16 converted on the way in: the
// reference's fused gate kernel takes 16-bit logits and computes in fp32,
// python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:44-46).
template <int VPL, int LT>
__device__ __forceinline__ void load_token_logits(const void* __restrict__ logits_v, int64_t token,
                                                  bool live, int E, int64_t ld, int vec_ok,
                                                  float (&v)[VPL]) {
  const int lane16 = threadIdx.x & 15;
  // every lane of a row takes the same branch; DPP rows never straddle tokens
  const float NEG_INF = -__builtin_inff();
  const int e0 = lane16 * VPL;
  if constexpr (LT == DLB_DTYPE_F32) {
    const float* logits = (const float*)logits_v;
    if (live && vec_ok) {
      const f32x4* p = reinterpret_cast<const f32x4*>(logits + token * ld + e0);
#pragma unroll
      for (int q = 0; q < VPL / 4; ++q) {
        const f32x4 t = p[q];
        v[4 * q + 0] = t[0];
        v[4 * q + 1] = t[1];
        v[4 * q + 2] = t[2];
        v[4 * q + 3] = t[3];
      }
    } else {
#pragma unroll
      for (int j = 0; j < VPL; ++j)
        v[j] = (live && e0 + j < E) ? logits[token * ld + e0 + j] : NEG_INF;
    }
  } else {
    const unsigned short* logits = (const unsigned short*)logits_v;
    if (live && vec_ok) {
      const unsigned short* p = logits + token * ld + e0;
      unsigned int w[VPL / 2];
      if constexpr (VPL == 4) {
        const u32x2 t = *reinterpret_cast<const u32x2*>(p);
        w[0] = t[0];
        w[1] = t[1];
      } else {
#pragma unroll
        for (int q = 0; q < VPL / 8; ++q) {
          const u32x4 t = reinterpret_cast<const u32x4*>(p)[q];
#pragma unroll
          for (int i = 0; i < 4; ++i) w[4 * q + i] = t[i];
        }
      }
#pragma unroll
      for (int q = 0; q < VPL / 2; ++q) {
        v[2 * q] = Elem<LT>::lo(w[q]);
        v[2 * q + 1] = Elem<LT>::hi(w[q]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < VPL; ++j)
        v[j] = (live && e0 + j < E) ? Elem<LT>::load1(logits, token * ld + e0 + j) : NEG_INF;
    }
  }
}

// Routes one token, whose logits the calling DPP row holds: lane r < K of the row stores the
// r-th selected probability and expert and gets that expert back (other lanes and dead rows: -1).
// probs / masks (either may be null) are the outputs in the form of the reference's fused gate
// kernel (python/dlBLAS/dlblas/kernels/topk_gating_fwd_part1.py:47-60): the full softmax row
// gates[token, :] and, for every selection round r, the one-hot row masks[r, token, :] (int64).
template <int VPL>
__device__ __forceinline__ int32_t route_token(const float (&v)[VPL], float* __restrict__ weights,
                                               int32_t* __restrict__ ids, int64_t token, bool live,
                                               int E, int K, int renorm,
                                               float* __restrict__ probs = nullptr,
                                               int64_t* __restrict__ masks = nullptr, int64_t T = 0) {
  const int lane16 = threadIdx.x & 15;
  const int e0 = lane16 * VPL;

  // softmax statistics: p_e = exp(l_e - max) / sum
  float mx = v[0];
#pragma unroll
  for (int j = 1; j < VPL; ++j) mx = fmaxf(mx, v[j]);
  mx = row16_max(mx);
  float ex[VPL];
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    ex[j] = expf(v[j] - mx);  // exp(-inf) = 0 for the padding experts
    sum += ex[j];
  }
  sum = row16_sum(sum);
  if (probs && live) {
#pragma unroll
    for (int j = 0; j < VPL; ++j)
      if (e0 + j < E) probs[token * E + e0 + j] = ex[j] / sum;  // the value a selected expert's weight has
  }

  // K rounds of arg-max over (orderable(logit), 256 - index): ties -> lowest index.
  // tag 0 means "no candidate"; real candidates carry tag = 256 - index >= 1.
  uint32_t key[VPL];
  uint32_t alive = 0u;
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    key[j] = orderable(v[j]);
    alive |= (e0 + j < E) ? (1u << j) : 0u;
  }

  float my_w = 0.0f;  // lane r keeps the r-th selected probability
  int32_t my_id = 0;
  float wsum = 0.0f;
  for (int r = 0; r < K; ++r) {
    uint32_t bk = 0u, bt = 0u;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      // strict '>' keeps the lowest index among equal keys inside the lane (j ascending)
      if (((alive >> j) & 1u) && (bt == 0u || key[j] > bk)) {
        bk = key[j];
        bt = (uint32_t)(256 - (e0 + j));
      }
    }
    row_step_max<kDppQuadXor1>(bk, bt);
    row_step_max<kDppQuadXor2>(bk, bt);
    row_step_max<kDppRowHalfMirror>(bk, bt);
    row_step_max<kDppRowMirror>(bk, bt);
    const int sel = 256 - (int)bt;  // winning expert, identical on all 16 lanes
    if (masks && live) {
#pragma unroll
      for (int j = 0; j < VPL; ++j)
        if (e0 + j < E) masks[((int64_t)r * T + token) * E + e0 + j] = (e0 + j == sel) ? 1 : 0;
    }
    float p = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      if (e0 + j == sel) {
        p = ex[j] / sum;
        alive &= ~(1u << j);
      }
    }
    // only the owner lane holds a non-zero p; x + 0 + ... + 0 == x, so the row sum is a
    // bit-exact broadcast.
    p = row16_sum(p);
    wsum += p;
    if (lane16 == r) {
      my_w = p;
      my_id = sel;
    }
  }
  if (live && lane16 < K) {
    const float w = renorm ? my_w / wsum : my_w;
    weights[token * K + lane16] = w;
    ids[token * K + lane16] = my_id;
    return my_id;
  }
  return -1;
}

template <int VPL, int LT>
__global__ __launch_bounds__(256) void moe_topk_softmax_kernel(
    const void* __restrict__ logits, float* __restrict__ weights, int32_t* __restrict__ ids,
    int64_t T, int E, int K, int64_t ld, int renorm, int vec_ok, float* __restrict__ probs,
    int64_t* __restrict__ masks) {
  const int64_t token = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  float v[VPL];
  load_token_logits<VPL, LT>(logits, token, token < T, E, ld, vec_ok, v);
  route_token<VPL>(v, weights, ids, token, token < T, E, K, renorm, probs, masks, T);
}

// The router fused with the first step of the expert alignment: a workgroup of 1024 threads
// routes 64 * PASSES consecutive tokens (64 per pass) and histograms the experts it selected
// in LDS, then writes one row of the alignment's [chunks, E] count table -- the row of the
// chunk made of exactly those tokens' K * 64 * PASSES flat routing slots.  Integer LDS adds
// only, so the row does not depend on the order of execution.
template <int VPL, int PASSES, int LT>
__global__ __launch_bounds__(1024) void moe_topk_softmax_count_kernel(
    const void* __restrict__ logits, float* __restrict__ weights, int32_t* __restrict__ ids,
    int64_t T, int E, int K, int64_t ld, int renorm, int vec_ok,
    int32_t* __restrict__ chunk_counts) {
  __shared__ int32_t hist[256];
  for (int e = threadIdx.x; e < E; e += 1024) hist[e] = 0;
  __syncthreads();
  const int64_t first = (int64_t)blockIdx.x * (64 * PASSES);
  float v[PASSES][VPL];
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {  // all loads first: one memory round trip
    const int64_t token = first + pass * 64 + (threadIdx.x >> 4);
    load_token_logits<VPL, LT>(logits, token, token < T, E, ld, vec_ok, v[pass]);
  }
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int64_t token = first + pass * 64 + (threadIdx.x >> 4);
    const int32_t e = route_token<VPL>(v[pass], weights, ids, token, token < T, E, K, renorm);
    if (e >= 0) atomicAdd(&hist[e], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 1024) chunk_counts[(int64_t)blockIdx.x * E + e] = hist[e];
}

// whole-row vector loads of the logits: 16-byte aligned base, rows a whole number of 16-byte pieces
bool logits_vector_ok(const void* logits, int dtype, int64_t ld) {
  return aligned16(logits) && ld % (dtype == DLB_DTYPE_F32 ? 4 : 8) == 0;
}

}  // namespace

// launch of the fused router + chunk histogram (used by the fused entry point of the alignment);
// chunk_tokens is 64 or 128
int launch_topk_softmax_count(const void* logits, int logits_dtype, float* weights, int32_t* ids,
                              int64_t T, int E, int K, int64_t ld_logits, int renormalize,
                              int chunk_tokens, int32_t* chunk_counts, hipStream_t s) {
  if (chunk_tokens != 64 && chunk_tokens != 128) return DLB_ERR_BAD_ARG;
  const dim3 grid((uint32_t)ceil_div(T, chunk_tokens)), block(1024);
  const bool a16 = logits_vector_ok(logits, logits_dtype, ld_logits);
#define DLB_LAUNCH_ROUTE_COUNT_LT(VPL_, EFULL_, LT_)                                               \
  do {                                                                                             \
    if (chunk_tokens == 64)                                                                        \
      hipLaunchKernelGGL((moe_topk_softmax_count_kernel<VPL_, 1, LT_>), grid, block, 0, s, logits, \
                         weights, ids, T, E, K, ld_logits, renormalize, (int)(a16 && E == EFULL_), \
                         chunk_counts);                                                            \
    else                                                                                           \
      hipLaunchKernelGGL((moe_topk_softmax_count_kernel<VPL_, 2, LT_>), grid, block, 0, s, logits, \
                         weights, ids, T, E, K, ld_logits, renormalize, (int)(a16 && E == EFULL_), \
                         chunk_counts);                                                            \
  } while (0)
#define DLB_LAUNCH_ROUTE_COUNT(VPL_, EFULL_)                                          \
  do {                                                                                \
    if (logits_dtype == DLB_DTYPE_F32) DLB_LAUNCH_ROUTE_COUNT_LT(VPL_, EFULL_, DLB_DTYPE_F32);      \
    else if (logits_dtype == DLB_DTYPE_BF16) DLB_LAUNCH_ROUTE_COUNT_LT(VPL_, EFULL_, DLB_DTYPE_BF16); \
    else DLB_LAUNCH_ROUTE_COUNT_LT(VPL_, EFULL_, DLB_DTYPE_F16);                                    \
  } while (0)
  if (E <= 64) DLB_LAUNCH_ROUTE_COUNT(4, 64);
  else if (E <= 128) DLB_LAUNCH_ROUTE_COUNT(8, 128);
  else DLB_LAUNCH_ROUTE_COUNT(16, 256);
#undef DLB_LAUNCH_ROUTE_COUNT
#undef DLB_LAUNCH_ROUTE_COUNT_LT
  return launch_status();
}

}  // namespace dlb

extern "C" int dlb_moe_topk_softmax_f32(const void* logits, float* weights, int32_t* ids,
                                        float* probs, int64_t* masks, int64_t T, int E, int K,
                                        int64_t ld_logits, int logits_dtype, int renormalize,
                                        void* stream) {
  using namespace dlb;
  if (T < 0 || E < 1 || K < 1 || K > E || ld_logits < E) return DLB_ERR_BAD_ARG;
  if (K > 16 || E > 256) return DLB_ERR_UNSUPPORTED;
  if (logits_dtype != DLB_DTYPE_F32 && logits_dtype != DLB_DTYPE_BF16 && logits_dtype != DLB_DTYPE_F16)
    return DLB_ERR_UNSUPPORTED;
  if (T == 0) return DLB_OK;
  if (!logits || !weights || !ids) return DLB_ERR_BAD_ARG;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)ceil_div(T, 16)), block(256);
  const bool a16 = logits_vector_ok(logits, logits_dtype, ld_logits);
#define DLB_LAUNCH_ROUTE(LT_)                                                                      \
  do {                                                                                             \
    if (E <= 64)                                                                                   \
      hipLaunchKernelGGL((moe_topk_softmax_kernel<4, LT_>), grid, block, 0, s, logits, weights, ids, \
                         T, E, K, ld_logits, renormalize, (int)(a16 && E == 64), probs, masks);    \
    else if (E <= 128)                                                                             \
      hipLaunchKernelGGL((moe_topk_softmax_kernel<8, LT_>), grid, block, 0, s, logits, weights, ids, \
                         T, E, K, ld_logits, renormalize, (int)(a16 && E == 128), probs, masks);   \
    else                                                                                           \
      hipLaunchKernelGGL((moe_topk_softmax_kernel<16, LT_>), grid, block, 0, s, logits, weights,   \
                         ids, T, E, K, ld_logits, renormalize, (int)(a16 && E == 256), probs,      \
                         masks);                                                                   \
  } while (0)
  if (logits_dtype == DLB_DTYPE_F32) DLB_LAUNCH_ROUTE(DLB_DTYPE_F32);
  else if (logits_dtype == DLB_DTYPE_BF16) DLB_LAUNCH_ROUTE(DLB_DTYPE_BF16);
  else DLB_LAUNCH_ROUTE(DLB_DTYPE_F16);
#undef DLB_LAUNCH_ROUTE
  return launch_status();
}
