// Fused SiLU-and-mul for gfx950: out[m, j] = silu(x[m, j]) * x[m, N + j].
//
// Follows the arithmetic of the reference Triton kernels
// (python/dlBLAS/dlblas/kernels/activation.py:38-47): both halves are widened to fp32,
// gate / (1 + exp(-gate)) * up, one rounding to the output type at the store.
//
// The op is a pure HBM stream (3 bytes moved per output byte), so the kernel is built around
// 128-bit accesses: each lane owns 16-byte vectors of gate and up (UNROLL pairs, all requested
// before the first use; one pair per lane and many resident waves turned out fastest), and the
// grid is flattened over M * N / VEC so that a row length that is not a multiple of the block
// (N = 11008 -> 1376 vectors) leaves no idle lanes.
#include "common.h"

namespace dlb {
namespace {

__device__ __forceinline__ float silu_mul(float g, float u) {
  // __expf -> v_exp_f32 with a pre-multiply; relative error ~1e-7 is invisible after the
  // rounding to 8 (bf16) or 11 (f16) significand bits, as in the reference's fast_expf.
  return g / (1.0f + __expf(-g)) * u;
}

template <int DT, int UNROLL>
__global__ __launch_bounds__(256) void silu_and_mul_vec16(const u32x4* __restrict__ x,
                                                          u32x4* __restrict__ out,
                                                          uint32_t total_vec, uint32_t vec_per_row,
                                                          uint32_t ldx_vec, uint32_t ldo_vec) {
  // x and out are addressed in 16-byte units; vec_per_row = N / 8.
  const uint32_t base = blockIdx.x * (256u * UNROLL) + threadIdx.x;
  u32x4 g[UNROLL], u[UNROLL];
  uint32_t oidx[UNROLL];
#pragma unroll
  for (int j = 0; j < UNROLL; ++j) {
    const uint32_t i = base + j * 256u;
    if (i < total_vec) {
      const uint32_t row = i / vec_per_row;
      const uint32_t col = i - row * vec_per_row;
      const size_t off = (size_t)row * ldx_vec + col;
      g[j] = __builtin_nontemporal_load(x + off);
      u[j] = __builtin_nontemporal_load(x + off + vec_per_row);
      oidx[j] = row * ldo_vec + col;
    }
  }
#pragma unroll
  for (int j = 0; j < UNROLL; ++j) {
    const uint32_t i = base + j * 256u;
    if (i < total_vec) {
      u32x4 r;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float a = silu_mul(Elem<DT>::lo(g[j][w]), Elem<DT>::lo(u[j][w]));
        const float b = silu_mul(Elem<DT>::hi(g[j][w]), Elem<DT>::hi(u[j][w]));
        r[w] = Elem<DT>::pack(a, b);
      }
      __builtin_nontemporal_store(r, out + oidx[j]);
    }
  }
}

__global__ __launch_bounds__(256) void silu_and_mul_f32_vec16(const f32x4* __restrict__ x,
                                                              f32x4* __restrict__ out,
                                                              uint32_t total_vec,
                                                              uint32_t vec_per_row,
                                                              uint32_t ldx_vec, uint32_t ldo_vec) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total_vec) return;
  const uint32_t row = i / vec_per_row;
  const uint32_t col = i - row * vec_per_row;
  const size_t off = (size_t)row * ldx_vec + col;
  const f32x4 g = __builtin_nontemporal_load(x + off);
  const f32x4 u = __builtin_nontemporal_load(x + off + vec_per_row);
  f32x4 r;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = g[w] / (1.0f + expf(-g[w])) * u[w];
  __builtin_nontemporal_store(r, out + (size_t)row * ldo_vec + col);
}

// Element-wise path for shapes the vector path cannot take (odd N, unaligned views).
template <int DT>
__global__ __launch_bounds__(256) void silu_and_mul_scalar(const void* __restrict__ x,
                                                           void* __restrict__ out, int64_t M,
                                                           int64_t N, int64_t ldx, int64_t ldo) {
  const int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t row = i / N, col = i - row * N;
    if constexpr (DT == DLB_DTYPE_F32) {
      const float g = ((const float*)x)[row * ldx + col];
      const float u = ((const float*)x)[row * ldx + N + col];
      ((float*)out)[row * ldo + col] = g / (1.0f + expf(-g)) * u;
    } else {
      const float g = Elem<DT>::load1(x, row * ldx + col);
      const float u = Elem<DT>::load1(x, row * ldx + N + col);
      Elem<DT>::store1(out, row * ldo + col, silu_mul(g, u));
    }
  }
}

template <int DT>
int launch_16bit(const void* x, void* out, int64_t M, int64_t N, int64_t ldx, int64_t ldo,
                 hipStream_t s) {
  constexpr int VEC = 8, UNROLL = 1;  // measured: 1 -> 85 us, 2 -> 86.5, 4 -> 91.5, 8 -> 98 at [8192, 2 x 11008]
  const int64_t total_vec = M * (N / VEC);
  const bool vec_ok = (N % VEC == 0) && (ldx % VEC == 0) && (ldo % VEC == 0) && aligned16(x) &&
                      aligned16(out) && total_vec < (int64_t)0xffffffffu - 256 * UNROLL &&
                      M * (ldx / VEC) < (int64_t)0xffffffffu && M * (ldo / VEC) < (int64_t)0xffffffffu;
  if (vec_ok) {
    const uint32_t blocks = (uint32_t)ceil_div(total_vec, 256 * UNROLL);
    hipLaunchKernelGGL((silu_and_mul_vec16<DT, UNROLL>), dim3(blocks), dim3(256), 0, s,
                       (const u32x4*)x, (u32x4*)out, (uint32_t)total_vec, (uint32_t)(N / VEC),
                       (uint32_t)(ldx / VEC), (uint32_t)(ldo / VEC));
  } else {
    const int64_t blocks = ceil_div(M * N, 256);
    hipLaunchKernelGGL((silu_and_mul_scalar<DT>), dim3((uint32_t)(blocks < 65536 ? blocks : 65536)),
                       dim3(256), 0, s, x, out, M, N, ldx, ldo);
  }
  return launch_status();
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_silu_and_mul(const void* x, void* out, int64_t M, int64_t N, int64_t ld_x,
                                int64_t ld_out, int dtype, void* stream) {
  using namespace dlb;
  if (M < 0 || N < 0 || ld_x < 2 * N || ld_out < N) return DLB_ERR_BAD_ARG;
  if (M == 0 || N == 0) return DLB_OK;
  if (!x || !out) return DLB_ERR_BAD_ARG;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DLB_DTYPE_BF16:
      return launch_16bit<DLB_DTYPE_BF16>(x, out, M, N, ld_x, ld_out, s);
    case DLB_DTYPE_F16:
      return launch_16bit<DLB_DTYPE_F16>(x, out, M, N, ld_x, ld_out, s);
    case DLB_DTYPE_F32: {
      const int64_t total_vec = M * (N / 4);
      const bool vec_ok = (N % 4 == 0) && (ld_x % 4 == 0) && (ld_out % 4 == 0) && aligned16(x) &&
                          aligned16(out) && total_vec < (int64_t)0xffffff00u &&
                          M * (ld_x / 4) < (int64_t)0xffffffffu;
      if (vec_ok) {
        hipLaunchKernelGGL(silu_and_mul_f32_vec16, dim3((uint32_t)ceil_div(total_vec, 256)),
                           dim3(256), 0, s, (const f32x4*)x, (f32x4*)out, (uint32_t)total_vec,
                           (uint32_t)(N / 4), (uint32_t)(ld_x / 4), (uint32_t)(ld_out / 4));
      } else {
        const int64_t blocks = ceil_div(M * N, 256);
        hipLaunchKernelGGL((silu_and_mul_scalar<DLB_DTYPE_F32>),
                           dim3((uint32_t)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, s, x,
                           out, M, N, ld_x, ld_out);
      }
      return launch_status();
    }
    default:
      return DLB_ERR_UNSUPPORTED;
  }
}
