// Measurement aids, not operators: what matrix-instruction rate does THIS chip sustain on given
// operand data, and what does a plain non-temporal stream reach?  The published MFMA peaks assume the 2.4 GHz boost clock; under matrix load the
// clock follows the power the data draws, so back-to-back MFMAs on random operands run well
// below the rate they reach on zeros.  The benchmark reports the kernels' rates beside this
// measured ceiling (and beside the published peak).
//
// Every wave cycles through four operand pairs read once from `operands` (so the registers hold
// the caller's data, whatever its entropy) and issues `iters` rounds of four independent MFMAs;
// no memory traffic or LDS inside the loop, and vector arithmetic only on request: with
// valu_per_mfma > 0 it measures how much of a wave's vector work the SIMD hides under its
// matrix instructions.
#include "../common.h"
#include "bench_probe.h"

namespace dlb {
namespace {

constexpr int kProbeThreads = 512;      // two waves per SIMD
constexpr int kProbeWordsPerLane = 64;  // 4 pairs x (two 16-byte halves of A and of B)

// NV > 0: every MFMA is followed by NV independent fp32 multiply-adds of the same wave (eight
// dependency chains), the mix of a kernel that does vector arithmetic between its matrix
// instructions; a scheduling fence after each group keeps the two kinds interleaved as written.
template <bool FP8, int NV>
__global__ __launch_bounds__(kProbeThreads) void mfma_rate_kernel(const uint32_t* __restrict__ data,
                                                                  float* sink, int iters) {
  u32x4 a[4], b[4], a2[4], b2[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t* p = data + ((size_t)(blockIdx.x * kProbeThreads + threadIdx.x) * 4 + i) * 16;
    a[i] = *(const u32x4*)p;
    b[i] = *(const u32x4*)(p + 4);
    a2[i] = *(const u32x4*)(p + 8);
    b2[i] = *(const u32x4*)(p + 12);
  }
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  float x[8];
#pragma unroll
  for (int f = 0; f < 8; ++f) x[f] = 1.0f + 0.001f * (float)((threadIdx.x + f) & 7);
  const float c1 = 1.0f - 1e-6f * (float)(iters & 1), c2 = 1e-6f * (float)(iters & 3);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (FP8) {
        const i32x8 x = {(int)a[i][0],  (int)a[i][1],  (int)a[i][2],  (int)a[i][3],
                         (int)a2[i][0], (int)a2[i][1], (int)a2[i][2], (int)a2[i][3]};
        const i32x8 y = {(int)b[i][0],  (int)b[i][1],  (int)b[i][2],  (int)b[i][3],
                         (int)b2[i][0], (int)b2[i][1], (int)b2[i][2], (int)b2[i][3]};
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, acc[i], 0, 0, 0, 0, 0, 0);
      } else {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i]),
                                                         __builtin_bit_cast(bf16x8, b[i]), acc[i],
                                                         0, 0, 0);
      }
      if (NV > 0) {
#pragma unroll
        for (int f = 0; f < NV; ++f) x[f & 7] = __builtin_fmaf(x[f & 7], c1, c2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float s = 0.0f;
#pragma unroll
  for (int f = 0; f < 8; ++f) s += x[f];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (s == 12345.678f) sink[threadIdx.x] = s;  // keeps the loop alive; practically never true
}

// Streaming ceiling: every lane reads 16-byte vectors with non-temporal loads, eight in flight per
// lane, and folds them into a value that is practically never stored.
__global__ __launch_bounds__(256) void hbm_read_kernel(const u32x4* __restrict__ src, float* sink,
                                                       uint64_t nvec) {
  constexpr int U = 8;
  const uint64_t base = (uint64_t)blockIdx.x * (256u * U) + threadIdx.x;
  unsigned int acc = 0;
#pragma unroll
  for (int j = 0; j < U; ++j) {
    const uint64_t i = base + (uint64_t)j * 256u;
    if (i < nvec) {
      const u32x4 v = __builtin_nontemporal_load(src + i);
      acc |= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
  }
  if (acc == 0x9e3779b9u) sink[threadIdx.x] = 1.0f;
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_probe_hbm_read(const void* src, void* sink, int64_t sink_bytes, int64_t bytes,
                                  void* stream) {
  using namespace dlb;
  if (bytes < 0 || !src || !sink) return DLB_ERR_BAD_ARG;
  if (sink_bytes < DLB_PROBE_SINK_BYTES) return DLB_ERR_WORKSPACE;
  if (bytes == 0) return DLB_OK;
  if (bytes % 16 != 0 || !aligned16(src)) return DLB_ERR_UNSUPPORTED;
  const uint64_t nvec = (uint64_t)bytes / 16;
  const uint64_t nblk = (nvec + 256 * 8 - 1) / (256 * 8);
  if (nblk > 0x7fffffffu) return DLB_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(hbm_read_kernel, dim3((uint32_t)nblk), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)src, (float*)sink, nvec);
  return launch_status();
}

extern "C" int64_t dlb_probe_mfma_operand_bytes(int blocks) {
  if (blocks < 1) return 0;
  return (int64_t)blocks * dlb::kProbeThreads * dlb::kProbeWordsPerLane * 4;
}

extern "C" int dlb_probe_mfma_rate(const void* operands, int64_t operand_bytes, void* sink,
                                   int64_t sink_bytes, int blocks, int fp8, int iters,
                                   int valu_per_mfma, void* stream) {
  using namespace dlb;
  if (blocks < 1 || iters < 0 || !operands || !sink) return DLB_ERR_BAD_ARG;
  if (valu_per_mfma != 0 && valu_per_mfma != 4 && valu_per_mfma != 8 && valu_per_mfma != 16)
    return DLB_ERR_UNSUPPORTED;
  if (sink_bytes < DLB_PROBE_SINK_BYTES) return DLB_ERR_WORKSPACE;
  if (operand_bytes < dlb_probe_mfma_operand_bytes(blocks)) return DLB_ERR_WORKSPACE;
  if (!aligned16(operands)) return DLB_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((uint32_t)blocks), dim3(kProbeThreads), 0, s,
                       (const uint32_t*)operands, (float*)sink, iters);
  };
  switch (valu_per_mfma + (fp8 ? 100 : 0)) {
    case 0: launch(mfma_rate_kernel<false, 0>); break;
    case 4: launch(mfma_rate_kernel<false, 4>); break;
    case 8: launch(mfma_rate_kernel<false, 8>); break;
    case 16: launch(mfma_rate_kernel<false, 16>); break;
    case 100: launch(mfma_rate_kernel<true, 0>); break;
    case 104: launch(mfma_rate_kernel<true, 4>); break;
    case 108: launch(mfma_rate_kernel<true, 8>); break;
    default: launch(mfma_rate_kernel<true, 16>); break;
  }
  return launch_status();
}
