// fp8 (OCP e4m3fn) per-token-group quantisation of activations, shared by the stand-alone
// quantiser and by the launch that runs it beside the expert alignment.
// Rule: per group of 128 consecutive elements of a row, scale = max(absmax, 1e-10) / 448 and
// q = rne_e4m3(clamp(x / scale, +-448)).
#pragma once
#include "common.h"

namespace dlb {

constexpr float kFp8Max = 448.0f;
constexpr float kQuantEps = 1e-10f;

__device__ __forceinline__ unsigned int pack4_fp8(float a, float b, float c, float d) {
  // v_cvt_pk_fp8_f32 rounds to nearest even; values beyond +-464 would become NaN, so clamp.
  a = fminf(fmaxf(a, -kFp8Max), kFp8Max);
  b = fminf(fmaxf(b, -kFp8Max), kFp8Max);
  c = fminf(fmaxf(c, -kFp8Max), kFp8Max);
  d = fminf(fmaxf(d, -kFp8Max), kFp8Max);
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (unsigned int)r;
}

constexpr int kQuantThreads = 256;
constexpr int kQuantUnroll = 4;  // groups per DPP row and workgroup pass (loads issued together)
constexpr int kQuantGroupsPerBlock = (kQuantThreads / 16) * kQuantUnroll;

struct QuantParams {
  const unsigned short* x;
  unsigned char* xq;
  float* xs;
  int64_t total_groups;
  int groups_per_row;
  int64_t ldx, ldq, lds;
};

// the work of workgroup `block` (kQuantThreads threads): one DPP row (16 lanes x 8 elements) per
// 128-element group, kQuantUnroll groups per row
template <int DT>
__device__ __forceinline__ void quant_fp8_group128_block(const QuantParams& q, int64_t block) {
  const int lane16 = threadIdx.x & 15;
  int64_t row[kQuantUnroll];
  int gc[kQuantUnroll];
  bool live[kQuantUnroll];
  u32x4 raw[kQuantUnroll];
#pragma unroll
  for (int u = 0; u < kQuantUnroll; ++u) {
    const int64_t gidx = (block * kQuantUnroll + u) * 16 + (threadIdx.x >> 4);
    live[u] = gidx < q.total_groups;
    row[u] = live[u] ? gidx / q.groups_per_row : 0;
    gc[u] = live[u] ? (int)(gidx - row[u] * q.groups_per_row) : 0;
    raw[u] = u32x4{0u, 0u, 0u, 0u};
    if (live[u]) raw[u] = __builtin_nontemporal_load((const u32x4*)(q.x + row[u] * q.ldx + gc[u] * 128 + lane16 * 8));
  }
#pragma unroll
  for (int u = 0; u < kQuantUnroll; ++u) {
    float v[8];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      v[2 * w] = Elem<DT>::lo(raw[u][w]);
      v[2 * w + 1] = Elem<DT>::hi(raw[u][w]);
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    amax = row16_max(amax);
    const float scale = fmaxf(amax, kQuantEps) / kFp8Max;
    if (live[u]) {
      u32x2 o;
      o[0] = pack4_fp8(v[0] / scale, v[1] / scale, v[2] / scale, v[3] / scale);
      o[1] = pack4_fp8(v[4] / scale, v[5] / scale, v[6] / scale, v[7] / scale);
      *(u32x2*)(q.xq + row[u] * q.ldq + gc[u] * 128 + lane16 * 8) = o;
      if (lane16 == 0) q.xs[row[u] * q.lds + gc[u]] = scale;
    }
  }
}

// argument checks of the quantiser (shared by its two entry points); fills `q` on DLB_OK
inline int fill_quant_params(QuantParams& q, const void* x, void* xq, float* xs, int64_t M, int K,
                             int64_t ld_x, int64_t ld_q, int64_t ld_s, int dtype) {
  if (M < 0 || K < 0 || ld_x < K || ld_q < K || ld_s < K / 128) return DLB_ERR_BAD_ARG;
  if (M > 0 && K > 0 && (!x || !xq || !xs)) return DLB_ERR_BAD_ARG;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
  if (K % 128 != 0 || ld_x % 8 != 0 || ld_q % 8 != 0 || !aligned16(x) ||
      (reinterpret_cast<uintptr_t>(xq) & 7u) != 0)
    return DLB_ERR_UNSUPPORTED;
  q.x = (const unsigned short*)x;
  q.xq = (unsigned char*)xq;
  q.xs = xs;
  q.groups_per_row = K / 128;
  q.total_groups = M * (int64_t)(K / 128);
  q.ldx = ld_x;
  q.ldq = ld_q;
  q.lds = ld_s;
  return DLB_OK;
}

}  // namespace dlb
