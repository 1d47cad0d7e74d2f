// fp8 (OCP e4m3fn) fused-MoE building blocks for gfx950:
//   * per-token-group activation quantisation (groups of 128 along K, fp32 scales);
//   * expert-grouped GEMM over block-aligned routing (64- or 128-row blocks, one expert per
//     block) on the 32x32x64 f8f6f4 MFMA, with the block scales applied per 128-deep K chunk:
//         acc += mfma(x_q[:, kc], w_q[:, kc]) * x_scale[row, kc] * w_scale[n / 128, kc]
//     in two flavours -- "gate_up" (A rows gathered by token, SiLU-and-mul and re-quantisation
//     of the intermediate fused into the epilogue) and "down" (routing weight applied, rows
//     scattered back to their (token, slot) position);
//   * the deterministic sum over the top-k slots.
//
// Pipeline shape and layouts follow the reference's bf16 fused_moe
// (python/dlBLAS/dlblas/kernels/fused_moe.py:296-376: sort by expert, grouped GEMM over
// w1 [E, 2I, H] with the gate rows first, activation, grouped GEMM over w2 [E, H, I] times
// the routing weight, sum over top-k; kernel :82-175).  The fp8 scheme itself has no
// counterpart there; its nearest precedent is the int8 per-token quantisation and
// scale-in-epilogue GEMM of python/dlBLAS/dlblas/kernels/w8a8.py:102-106,275-335.
//
// The same kernels also run unquantised bf16/f16 operands (QT = 1): the reference's own
// fused_moe, with 32x32x16 MFMAs accumulating in place and no scales.
//
// GEMM mapping.  The MFMA runs "transposed": weight rows are the A operand (M index = output
// column n), activations the B operand (N index = token row), so a lane's sixteen accumulator
// registers of a 32x32 tile are 4 x 4 consecutive n of ONE token: the activation scale is a
// per-lane scalar and the epilogues store runs of adjacent outputs.  In the 64-row kernel
// weight fragments go straight from HBM/L2 into operand registers (each wave owns its own n
// range, so nothing is shared between waves) and only the 64 x 128-byte activation chunk
// passes through LDS; the 128-row kernel stages both operands in LDS.
#include <type_traits>

#include "common.h"

namespace dlb {
namespace {

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

// ---------------------------------------------------------------------------------------
// per-token-group quantisation: one DPP row (16 lanes x 8 elements) per 128-element group
// ---------------------------------------------------------------------------------------
constexpr int kQuantUnroll = 4;  // groups per DPP row and workgroup pass (loads issued together)

template <int DT>
__global__ __launch_bounds__(256) void quant_fp8_group128_kernel(
    const unsigned short* __restrict__ x, unsigned char* __restrict__ xq, float* __restrict__ xs,
    int64_t total_groups, int groups_per_row, int64_t ldx, int64_t ldq, int64_t lds) {
  const int lane16 = threadIdx.x & 15;
  int64_t row[kQuantUnroll];
  int gc[kQuantUnroll];
  bool live[kQuantUnroll];
  u32x4 raw[kQuantUnroll];
#pragma unroll
  for (int u = 0; u < kQuantUnroll; ++u) {
    const int64_t gidx = ((int64_t)blockIdx.x * kQuantUnroll + u) * 16 + (threadIdx.x >> 4);
    live[u] = gidx < total_groups;
    row[u] = live[u] ? gidx / groups_per_row : 0;
    gc[u] = live[u] ? (int)(gidx - row[u] * groups_per_row) : 0;
    raw[u] = u32x4{0u, 0u, 0u, 0u};
    if (live[u]) raw[u] = __builtin_nontemporal_load((const u32x4*)(x + row[u] * ldx + gc[u] * 128 + lane16 * 8));
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
      u32x2 q;
      q[0] = pack4_fp8(v[0] / scale, v[1] / scale, v[2] / scale, v[3] / scale);
      q[1] = pack4_fp8(v[4] / scale, v[5] / scale, v[6] / scale, v[7] / scale);
      *(u32x2*)(xq + row[u] * ldq + gc[u] * 128 + lane16 * 8) = q;
      if (lane16 == 0) xs[row[u] * lds + gc[u]] = scale;
    }
  }
}

// ---------------------------------------------------------------------------------------
// grouped GEMM
// ---------------------------------------------------------------------------------------
struct MoeGemmParams {
  const unsigned char* a;     // activations fp8 [rows, K]
  const float* a_scale;       // [rows, K / 128]
  const unsigned char* w;     // weights fp8 [E_local, N, K]
  const float* w_scale;       // [E_local, N / 128, K / 128]
  const int32_t* sorted_ids;  // [num_mblocks * BM]
  const int32_t* expert_ids;  // [num_mblocks]
  int num_mblocks, num_ntiles, grid_real;
  int K, N, KC;               // K = bytes per activation / weight row, KC = K / 128
  int topk, numel;            // flat slots = tokens * topk (also the pad sentinel)
  int num_tokens;
  int expert_offset;          // weights hold experts [expert_offset, expert_offset + E_local)
  int num_local;              // E_local
  int w_layout;               // 0: [E, N, K] row-major, 1: MFMA-operand order (see header)
  // gate_up flavour
  unsigned char* hq;          // [num_mblocks * BM, I] fp8, or 16-bit when QT = 1
  float* hs;                  // [num_mblocks * BM, I / 128]
  int I;
  // down flavour
  void* out;                  // [numel, N] bf16/f16
  const float* topk_w;        // [numel]
};


// QT = 0: fp8 operands with block scales; QT = 1: 16-bit operands of type DT, no scales.
// GATED = true : gate_up GEMM (N = 2I), tile = 128 gate cols + the matching 128 up cols,
//                epilogue silu(gate) * up -> fp8 + per-128 scale, rows kept in sorted order.
// GATED = false: down GEMM, tile = 256 cols, epilogue * routing weight -> out[slot, n].
// WL = weight layout (0 row-major, 1 operand order).  64 rows (routing slots) per workgroup.
//
// MFMA shape: 32x32x64 (fp8) / 32x32x16 (16 bit).  A wave owns 64 output columns (two 32-column
// tiles; gated: 32 gate + the matching 32 up columns) x the 64 rows (two 32-row tiles).  Lane
// (j = lane % 32, h = lane / 32) supplies, for weight row / token j, the four 16-byte pieces
// q = 0..3 of a 128-byte K chunk at chunk offset 32 q + 16 h; the fp8 MFMA m consumes pieces
// 2m and 2m + 1, the 16-bit MFMA q consumes piece q.  Its 16 accumulators of a tile are
// token j, columns 8 (r / 4) + 4 h + r % 4.  The 32x32 shape matters for the fp8 path: next to
// an fp8 32x32x64 MFMA (64 cycles) the vector ALU retires the 8 scale-and-accumulate FMAs it
// owes per MFMA at ~94 % matrix-pipe occupancy, next to the 16x16x128 form (32 cycles, 4 FMAs)
// only at ~70 %.
//
// Data movement, all of it issued by hand so that nothing waits for more than it needs (the
// compiler's wait-count pass treats a load under a run-time condition as possibly absent and
// then waits for everything younger too, which defeats a deep prefetch):
//   * weights: global -> operand registers in units of (chunk, column tile) = 4 x 16 bytes per
//     lane, a ring of four units, each refilled right after its last use for the chunk after
//     next (1.5 chunks ahead);
//   * activations: global -> LDS directly (three chunk slots of 64 x 128 bytes, rows swizzled
//     by (row >> 1) & 7 in 16-byte pieces), issued two chunks ahead; one barrier per chunk, in
//     the middle of its MFMAs, publishes the next chunk; the scales of a chunk travel with it
//     (one 4-byte copy per wave: the activation scales of its 16 staging rows and its own
//     block scales);
//   * every wave issues the same number of loads per chunk (chunks past K re-load clamped or
//     dummy addresses), so the explicit vmcnt waits are compile-time constants.
#ifndef DLB_MOE_OCC
#define DLB_MOE_OCC 2
#endif


__device__ __forceinline__ i32x8 cat8(const u32x4& lo, const u32x4& hi) {
  return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
               (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

// exchange between the two lane halves: afterwards lane half 0 holds (its a, the partner's a)
// and lane half 1 (the partner's b, its b), partner = the lane 32 away
__device__ __forceinline__ void swap_halves(unsigned int& a, unsigned int& b) {
  typedef __attribute__((ext_vector_type(2))) unsigned int u2;
  const u2 r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

// one weight unit: the lane's four 16-byte pieces, uniform base + 32-bit lane offset
template <int WL>
__device__ __forceinline__ void load_w_unit(u32x4 (&b)[4], unsigned int voff, const unsigned char* sbase) {
  if constexpr (WL != 0)
    asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                 "global_load_dwordx4 %1, %4, %5 offset:512\n\t"
                 "global_load_dwordx4 %2, %4, %5 offset:1024\n\t"
                 "global_load_dwordx4 %3, %4, %5 offset:1536"
                 : "=&v"(b[0]), "=&v"(b[1]), "=&v"(b[2]), "=&v"(b[3])
                 : "v"(voff), "s"(sbase)
                 : "memory");
  else
    asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                 "global_load_dwordx4 %1, %4, %5 offset:32\n\t"
                 "global_load_dwordx4 %2, %4, %5 offset:64\n\t"
                 "global_load_dwordx4 %3, %4, %5 offset:96"
                 : "=&v"(b[0]), "=&v"(b[1]), "=&v"(b[2]), "=&v"(b[3])
                 : "v"(voff), "s"(sbase)
                 : "memory");
}
// wait until at most N vector-memory operations are outstanding; the unit's registers are
// tied to the wait so that nothing reads them earlier
template <int N>
__device__ __forceinline__ void wait_w_unit(u32x4 (&b)[4]) {
  asm volatile("s_waitcnt vmcnt(%4)" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <bool GATED, int DT, int QT, int WL>
__device__ __forceinline__ void moe_gemm_fp8_tile(const MoeGemmParams& p, const int logical) {
  constexpr int BM = 64;
  constexpr int NX = 3;                 // activation chunk slots in LDS
  constexpr int kXSlot = BM * 128;      // bytes of one slot
  constexpr int kScWave = 80;           // scale strip of a wave per slot: its 16 x-scales, its w-scales
  constexpr int kScSlot = 4 * kScWave;
  constexpr int D = QT == 0 ? 3 : 2;    // direct-to-LDS operations per wave and chunk
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds[NX * kXSlot];
  __shared__ __attribute__((aligned(16))) unsigned char sc_lds[NX * kScSlot];
  __shared__ float red_lds[4][BM];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int j = lane & 31;
  const int drow = lane >> 3, dpc = lane & 7;
  const int mb = logical % p.num_mblocks;
  const int nt = logical / p.num_mblocks;
  const int row0 = mb * BM;
  const int K = p.K, KC = p.KC;

  // The routing slots this lane needs are requested together with the block's expert id, so the
  // prologue pays one memory round trip for its metadata, not two.  Gated: the rows the lane
  // stages (two) and the row whose scale it fetches.  Down: the lane's two output rows and
  // their routing weights (first touched in the epilogue; the loads are older than everything
  // the main loop issues).
  int meta_sid[3] = {0, 0, 0};
  if (GATED) {
    meta_sid[0] = p.sorted_ids[row0 + 16 * wave + drow];
    meta_sid[1] = p.sorted_ids[row0 + 16 * wave + 8 + drow];
    meta_sid[2] = p.sorted_ids[row0 + 16 * wave + (lane & 15)];
  } else {
    meta_sid[0] = p.sorted_ids[row0 + j];
    meta_sid[1] = p.sorted_ids[row0 + 32 + j];
  }
  const int e_global = p.expert_ids[mb];
  const int e = e_global - p.expert_offset;
  if (e_global < 0 || e < 0 || e >= p.num_local) return;  // tail block / expert of another shard

  int out_sid[2] = {0, 0};
  float out_rw[2] = {0.0f, 0.0f};
  if (!GATED) {
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      out_sid[rt] = meta_sid[rt];
      out_rw[rt] = out_sid[rt] < p.numel ? p.topk_w[out_sid[rt]] : 0.0f;
    }
  }
  // source row of staging row i (gated: the slot's token; pad slots read a valid row)
  auto src_row_of = [&](int which, int r) -> int64_t {
    if (GATED) return min(meta_sid[which] / p.topk, p.num_tokens - 1);
    return row0 + r;
  };
  // ---- activation staging: per chunk 8 instructions of 8 rows x 128 bytes, two per wave;
  // lane -> (row, physical piece), the logical piece it fetches undoes the swizzle
  const unsigned char* xsrc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = 16 * wave + 8 * i + drow;
    xsrc[i] = p.a + src_row_of(i, r) * K + ((dpc ^ ((r >> 1) & 7)) << 4);
  }
  // scales: one 4-byte copy per wave and chunk with 18 lanes active: lanes 0..15 fetch the
  // activation scales of the wave's 16 staging rows, lanes 16 / 17 the block scale of the wave's
  // column tile 0 / 1
  const float* scsrc = nullptr;

  // ---- weight fragments: column tile ct of this wave covers 32 output columns
  int ncol[2];  // first column of tile ct in the expert's [N, K] matrix
  if (GATED) {
    ncol[0] = nt * 128 + wave * 32;
    ncol[1] = p.I + ncol[0];
  } else {
    ncol[0] = nt * 256 + wave * 64;
    ncol[1] = ncol[0] + 32;
  }
  const unsigned char* wbase = p.w + (int64_t)e * p.N * K;
  constexpr int kWChunk = WL ? 2048 : 128;  // byte distance between consecutive K chunks
  uint32_t woff[2];
  const float* wssrc = nullptr;
#pragma unroll
  for (int ct = 0; ct < 2; ++ct) {
    if (WL) {
      // operand-order storage: per (16-row group, chunk) one 2 KB block = [piece pair][16-byte
      // piece g][row c][16 B] holding K bytes 64 (pair) + 16 g; lane (j, h) takes pieces
      // g = 2 (q & 1) + h of pair q >> 1: every load covers two contiguous 512-byte runs
      const int nb = min((ncol[ct] >> 4) + (j >> 4), (p.N >> 4) - 1);
      woff[ct] = (uint32_t)nb * (uint32_t)KC * 2048u + (uint32_t)h * 256u + (uint32_t)(j & 15) * 16u;
    } else {
      const int n = min(ncol[ct] + j, p.N - 1);
      woff[ct] = (uint32_t)n * (uint32_t)K + 16u * h;
    }
  }
  if (QT == 0) {
    const int ct = GATED ? (lane == 17 ? 1 : 0) : 0;
    const int sblk = min(ncol[ct] >> 7, (p.N >> 7) - 1);
    scsrc = lane < 16 ? p.a_scale + src_row_of(2, 16 * wave + (lane & 15)) * KC
                      : p.w_scale + ((int64_t)e * (p.N >> 7) + sblk) * KC;
  }

  const unsigned int x_dst0 = lds_addr(x_lds) + wave * 2048;
  const unsigned int sc_dst0 = lds_addr(sc_lds) + wave * kScWave;
  // all direct-to-LDS operations of chunk kc (clamped past the end: the count per chunk is fixed)
  auto issue_x = [&](int kc, int slot) {
    const int kcc = min(kc, KC - 1);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      dma16_global_to_lds(xsrc[i] + kcc * 128, x_dst0 + slot * kXSlot + i * 1024);
    if constexpr (QT == 0) {
      dma4_global_to_lds_masked<0x3ffffull>(scsrc + kcc, sc_dst0 + slot * kScSlot);
    }
  };
  // weight unit (kc, ct); past the end every lane re-reads the expert's first 16 bytes
  auto issue_w = [&](int kc, int ct, u32x4 (&b)[4]) {
    const bool live = kc < KC;
    const unsigned char* sbase = uniform_ptr(wbase + (live ? kc : 0) * kWChunk);
    load_w_unit<WL>(b, live ? woff[ct] : 0u, sbase);
  };

  // ---- fragment reads of the activations: lane (j, h), row tile rt, pieces 2q + h at
  // physical piece (2q + h) ^ ((j >> 1) & 7): byte offsets f0 ^ (32 q)
  const int f0 = j * 128 + (((h ^ (j >> 1)) & 7) << 4);
  int xf[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) xf[q] = f0 ^ (q << 5);
  // row r's scale sits at (r / 16) * kScWave + (r % 16) * 4 of a slot; rows j and 32 + j are
  // two waves' strips apart
  const unsigned char* as_mine = sc_lds + (j >> 4) * kScWave + (j & 15) * 4;
  const unsigned char* ws_mine = sc_lds + wave * kScWave + 64;
  auto read_x = [&](int slot, int rt, u32x4 (&x)[4], float& as) {
#pragma unroll
    for (int q = 0; q < 4; ++q) x[q] = *(const u32x4*)(x_lds + slot * kXSlot + rt * 4096 + xf[q]);
    as = QT == 0 ? *(const float*)(as_mine + slot * kScSlot + rt * (2 * kScWave)) : 1.0f;
  };

  f32x16 acc[2][2];  // [row tile][column tile]
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][ct][r] = 0.0f;
  f32x16 pp;
#pragma unroll
  for (int r = 0; r < 16; ++r) pp[r] = 0.0f;
  float psc = 0.0f;

  u32x4 wr[2][2][4];   // weight units [chunk parity][column tile]
  u32x4 x0[4], x1[4];  // activation fragments of row tile 0 / 1
  float as0 = 1.0f, as1 = 1.0f;

  // one (row tile, column tile) step: the chunk's MFMAs, each followed by its share of the FMAs
  // that retire the previous step's product into `prev`
  auto step = [&](const u32x4 (&b)[4], const u32x4 (&x)[4], f32x16& own, f32x16& prev, float sc) {
    if constexpr (QT == 0) {
      (void)own;
      f32x16 pc;
#pragma unroll
      for (int r = 0; r < 16; ++r) pc[r] = 0.0f;
      pc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cat8(b[0], b[1]), cat8(x[0], x[1]), pc, 0,
                                                           0, 0, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 8; ++r) prev[r] += pp[r] * psc;
      // keep the retiring FMAs inside this step (the optimiser would otherwise sink them into
      // one long VALU run with nothing to overlap)
      asm volatile("" : "+v"(prev));
      pc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cat8(b[2], b[3]), cat8(x[2], x[3]), pc, 0,
                                                           0, 0, 0, 0, 0);
#pragma unroll
      for (int r = 8; r < 16; ++r) prev[r] += pp[r] * psc;
      asm volatile("" : "+v"(prev));
      pp = pc;
      psc = sc;
    } else {
      (void)prev;
      (void)sc;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if constexpr (DT == DLB_DTYPE_BF16)
          own = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[q]),
                                                        __builtin_bit_cast(bf16x8, x[q]), own, 0, 0, 0);
        else
          own = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b[q]),
                                                       __builtin_bit_cast(f16x8, x[q]), own, 0, 0, 0);
      }
    }
  };

  // Order of the vector-memory operations of a wave: X(0); then per chunk k = -2, -1, 0, ...
  //   W(k + 2, ct 0) [4]   X(k + 3) [D]   W(k + 2, ct 1) [4]
  // (the prologue plays chunks -2 and -1).  Operations complete in order, so "at most n
  // outstanding" means everything but the youngest n has landed.
  issue_x(0, 0);
  issue_w(0, 0, wr[0][0]);
  issue_x(1, 1);
  issue_w(0, 1, wr[0][1]);
  issue_w(1, 0, wr[1][0]);
  issue_x(2, 2);
  issue_w(1, 1, wr[1][1]);
  wait_vm<16 + 2 * D>();  // X(0) landed
  __syncthreads();
  read_x(0, 0, x0, as0);

  int x_cur = 0, x_nxt = 1, x_tgt = 2;  // slots of chunks k, k + 1, k + 2
  // Chunk k (P = k & 1), steps (ct 0, rt 0), (ct 0, rt 1), barrier, (ct 1, rt 0), (ct 1, rt 1).
  // On entry x0 = X(k, rt 0) is in registers.
  auto do_chunk = [&](auto ptag, int k) {
    constexpr int P = decltype(ptag)::value;
    float ws0 = 1.0f, ws1 = 1.0f;
    read_x(x_cur, 1, x1, as1);
    if constexpr (QT == 0) {
      ws0 = *(const float*)(ws_mine + x_cur * kScSlot);
      ws1 = GATED ? *(const float*)(ws_mine + x_cur * kScSlot + 4) : ws0;
    }
    wait_w_unit<12 + 2 * D>(wr[P][0]);  // W(k, ct 0) landed
    __builtin_amdgcn_sched_barrier(0);
    step(wr[P][0], x0, acc[0][0], acc[1][1], as0 * ws0);
    __builtin_amdgcn_sched_barrier(0);
    step(wr[P][0], x1, acc[1][0], acc[0][0], as1 * ws0);
    __builtin_amdgcn_sched_barrier(0);
    issue_w(k + 2, 0, wr[P][0]);
    wait_vm<16 + D>();  // this wave's part of X(k + 1) landed
    __syncthreads();    // X(k + 1) complete; every wave is done reading X(k)
    issue_x(k + 3, x_cur);
    wait_w_unit<12 + 2 * D>(wr[P][1]);  // W(k, ct 1) landed
    __builtin_amdgcn_sched_barrier(0);
    step(wr[P][1], x0, acc[0][1], acc[1][0], as0 * ws1);
    __builtin_amdgcn_sched_barrier(0);
    read_x(x_nxt, 0, x0, as0);
    __builtin_amdgcn_sched_barrier(0);
    step(wr[P][1], x1, acc[1][1], acc[0][1], as1 * ws1);
    __builtin_amdgcn_sched_barrier(0);
    issue_w(k + 2, 1, wr[P][1]);
    const int xr = x_cur;
    x_cur = x_nxt;
    x_nxt = x_tgt;
    x_tgt = xr;
  };
  for (int k = 0; k < KC; k += 2) {
    do_chunk(std::integral_constant<int, 0>{}, k);
    if (k + 1 < KC) do_chunk(std::integral_constant<int, 1>{}, k + 1);
  }
  // The clamped loads past the end are still in flight and will write the ring's registers:
  // the wait names those registers, so nothing after it can be given one of them earlier.
  asm volatile("s_waitcnt vmcnt(0)"
               : "+v"(wr[0][0][0]), "+v"(wr[0][0][1]), "+v"(wr[0][0][2]), "+v"(wr[0][0][3]),
                 "+v"(wr[0][1][0]), "+v"(wr[0][1][1]), "+v"(wr[0][1][2]), "+v"(wr[0][1][3]),
                 "+v"(wr[1][0][0]), "+v"(wr[1][0][1]), "+v"(wr[1][0][2]), "+v"(wr[1][0][3]),
                 "+v"(wr[1][1][0]), "+v"(wr[1][1][1]), "+v"(wr[1][1][2]), "+v"(wr[1][1][3])
               :
               : "memory");
  // retire the product of the very last step
  if constexpr (QT == 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[1][1][r] += pp[r] * psc;
  }


  // ---- epilogues: lane holds token (32*rt + j), columns ncol[ct] + 8*(r/4) + 4*h + r%4.
  // A swap between the lane halves turns two 4-column runs into one 8-column run per lane.
  if (GATED && QT == 1) {
    // rounding points of the reference pipeline (fused_moe.py:166,351-352): GEMM result,
    // silu(gate) and the product are each rounded to the activation type.  The 64 x 128 tile
    // is staged in the activation slots and leaves as whole 256-byte rows.
    constexpr int kActPitch = 256 + 16;
    static_assert(BM * kActPitch <= NX * kXSlot, "output staging fits the activation slots");
    __syncthreads();  // every wave is done reading the activation slots
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      unsigned short* dst = (unsigned short*)(x_lds + (32 * rt + j) * kActPitch) + wave * 32 + 8 * h;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        unsigned int o[2][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float v[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r = 4 * (2 * pr + s) + i;
            const unsigned int gu = Elem<DT>::pack(acc[rt][0][r], acc[rt][1][r]);
            const float gate = Elem<DT>::lo(gu), up = Elem<DT>::hi(gu);
            const float sg = Elem<DT>::lo(Elem<DT>::pack(gate / (1.0f + __expf(-gate)), 0.0f));
            v[i] = sg * up;
          }
          o[s][0] = Elem<DT>::pack(v[0], v[1]);
          o[s][1] = Elem<DT>::pack(v[2], v[3]);
        }
        swap_halves(o[0][0], o[1][0]);
        swap_halves(o[0][1], o[1][1]);
        *(u32x4*)(dst + 16 * pr) = u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // 64 rows x 16 pieces of 16 bytes, adjacent lanes on one row
      const int r = (tid >> 4) + 16 * i, pc = tid & 15;
      *(u32x4*)((unsigned short*)p.hq + (int64_t)(row0 + r) * p.I + nt * 128 + 8 * pc) =
          *(const u32x4*)(x_lds + r * kActPitch + 16 * pc);
    }
  } else if (GATED) {
    constexpr int kGatedPitch = 128 + 16;  // staging row pitch of the fp8 output tile
    float hv[2][16];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float amax = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float gate = acc[rt][0][r];
        const float up = acc[rt][1][r];
        const float v = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;  // 1-ulp reciprocal
        hv[rt][r] = v;
        amax = fmaxf(amax, fabsf(v));
      }
      amax = max_xor32(amax);
      if (h == 0) red_lds[wave][32 * rt + j] = amax;
    }
    __syncthreads();
    const int scol = nt;  // 128-column group index of the intermediate
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int r = 32 * rt + j;
      const float m = fmaxf(fmaxf(red_lds[0][r], red_lds[1][r]), fmaxf(red_lds[2][r], red_lds[3][r]));
      const float scale = fmaxf(m, kQuantEps) / kFp8Max;
      const float inv = __builtin_amdgcn_rcpf(scale);  // the stored scale stays exact
      const int64_t orow = row0 + r;
      unsigned int q[4];
#pragma unroll
      for (int s = 0; s < 4; ++s)
        q[s] = pack4_fp8(hv[rt][4 * s] * inv, hv[rt][4 * s + 1] * inv, hv[rt][4 * s + 2] * inv,
                         hv[rt][4 * s + 3] * inv);
      swap_halves(q[0], q[1]);
      swap_halves(q[2], q[3]);
      // staged in the activation slots (free: the barrier above came after every wave's main
      // loop) so that the tile leaves as whole 128-byte rows
      unsigned char* dst = x_lds + r * kGatedPitch + wave * 32 + 8 * h;
      *(u32x2*)(dst) = u32x2{q[0], q[1]};
      *(u32x2*)(dst + 16) = u32x2{q[2], q[3]};
      if (wave == 0 && h == 0) p.hs[orow * (p.I >> 7) + scol] = scale;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {  // 64 rows x 8 pieces of 16 bytes, adjacent lanes on one row
      const int r = (tid >> 3) + 32 * i, pc = tid & 7;
      *(u32x4*)(p.hq + (int64_t)(row0 + r) * p.I + nt * 128 + 16 * pc) =
          *(const u32x4*)(x_lds + r * kGatedPitch + 16 * pc);
    }
  } else {
    // The 64 x 256 output tile goes out through LDS, one 32-row half at a time (the activation
    // slots are free once every wave has left the main loop): a lane holds 16-byte runs of 32
    // different rows, the staged copy writes whole 512-byte rows with adjacent lanes on adjacent
    // 16-byte pieces.
    constexpr int kPitch = 512 + 16;  // staging row pitch: rows 16 bytes apart in the banks
    static_assert(32 * kPitch <= NX * kXSlot, "output staging fits the activation slots");
    unsigned char* stage = x_lds;
    const int ncols = min(256, p.N - nt * 256);  // multiple of 128
    __syncthreads();  // every wave is done reading the activation slots
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const float rw = out_rw[rt];
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) {
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
          unsigned int o[2][2];
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int r = 4 * (2 * pr + s);
            o[s][0] = Elem<DT>::pack(acc[rt][ct][r] * rw, acc[rt][ct][r + 1] * rw);
            o[s][1] = Elem<DT>::pack(acc[rt][ct][r + 2] * rw, acc[rt][ct][r + 3] * rw);
          }
          swap_halves(o[0][0], o[1][0]);
          swap_halves(o[0][1], o[1][1]);
          *(u32x4*)(stage + j * kPitch + (wave * 64 + ct * 32 + 16 * pr + 8 * h) * 2) =
              u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
        }
      }
      __syncthreads();
      // 32 rows x 32 pieces; thread t takes piece t % 32 of rows t / 32 + 8 i.  Row r's slot id
      // sits in lane r of every wave.
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = (tid >> 5) + 8 * i, pc = tid & 31;
        const int sid = __shfl(out_sid[rt], r);
        if (sid < p.numel && 8 * pc < ncols)
          *(u32x4*)((unsigned short*)p.out + (int64_t)sid * p.N + nt * 256 + 8 * pc) =
              *(const u32x4*)(stage + r * kPitch + 16 * pc);
      }
      if (rt == 0) __syncthreads();  // the second half reuses the staging rows
    }
  }
}

// Workgroup ids are dealt round-robin to the 8 XCDs, so XCD x takes the contiguous range
// [x * per_xcd, (x + 1) * per_xcd) of the logical tile order (same column tile, consecutive
// row blocks = mostly the same expert: neighbours share an L2) and its workgroups take
// consecutive tiles of it.  With fewer workgroups than tiles (a resident launch, two per CU)
// every workgroup walks a fixed sequence of tiles; with one workgroup per tile the loop runs
// once.
template <bool GATED, int DT, int QT, int WL>
__global__ __launch_bounds__(256, DLB_MOE_OCC) void moe_gemm_fp8_kernel(const MoeGemmParams p) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int per_xcd = (p.grid_real + 7) >> 3;
  for (int i = slot; i < per_xcd; i += slots) {
    const int logical = xcd * per_xcd + i;
    if (logical < p.grid_real) moe_gemm_fp8_tile<GATED, DT, QT, WL>(p, logical);
    __syncthreads();  // the tile's LDS is reused by the next one
  }
}

// ---------------------------------------------------------------------------------------
// Wide grouped GEMM: 128 routing slots x 256 output columns per workgroup of 8 waves (one
// workgroup per CU).  Twice the rows per weight byte of the 64-row kernel, which is what the
// L2 -> CU path rewards.  Both operands go HBM/L2 -> LDS with direct-to-LDS loads (no staging
// registers, no ds_write): per 128-byte K chunk 256 weight rows + 128 activation rows, each
// row 128 bytes with its eight 16-byte pieces XOR-swizzled by (row >> 1) & 7 so that the
// ds_read_b128 of an MFMA fragment (16 rows x 2 pieces per lane) runs at full LDS rate.
// Rings: weights 3 slots (issued two chunks ahead of use), activations 3 slots (one chunk
// ahead).  Wave (rg, cg) owns rows 64*rg.. and 64 columns; per chunk it reads its 4 weight
// fragments once (double-buffered in registers, fetched half a chunk early) and one
// activation fragment per 16-row step.  One barrier per chunk, placed in the middle of the
// chunk's MFMAs so nobody waits for LDS right after it.
// Weights may be row-major (8 lanes fetch one row's 128-byte line) or operand-order.
// ---------------------------------------------------------------------------------------
template <bool GATED, int DT, int QT>
__device__ __forceinline__ void moe_gemm_wide_tile(const MoeGemmParams& p, const int logical) {
  constexpr int BM = 128, BN = 256;
  constexpr int kWSlot = BN * 128;  // bytes of one weight ring slot
  constexpr int kXSlot = BM * 128;  // bytes of one activation ring slot
  constexpr int kSC = 16;           // chunks of activation scales resident in LDS
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds[3 * kWSlot];
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds[3 * kXSlot];
  __shared__ float as_lds[kSC][BM];
  __shared__ float ws_lds[2][kSC];  // block scales of the tile's two 128-column weight blocks
  __shared__ float red_lds[4][BM];
  __shared__ int32_t sid_lds[BM];

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave id, kept in scalar registers
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int j = lane & 31;
  const int rg = w >> 2;  // waves w and w + 4 share a SIMD: give them different row groups
  const int cg = w & 3;
  const int drow = lane >> 3, dpc = lane & 7;
  const int mb = logical % p.num_mblocks;
  const int nt = logical / p.num_mblocks;
  const int row0 = mb * BM;
  const int K = p.K, KC = p.KC;

  // the routing slots this thread needs (row tid % 128 for the slot list and the scales, the two
  // rows it stages) are requested together with the block's expert id: one round trip, not two
  const int sid_mine = p.sorted_ids[row0 + (tid & (BM - 1))];
  int sid_x[2] = {0, 0};
  if (GATED) {
    sid_x[0] = p.sorted_ids[row0 + 16 * w + drow];
    sid_x[1] = p.sorted_ids[row0 + 16 * w + 8 + drow];
  }
  const int e_global = p.expert_ids[mb];
  const int e = e_global - p.expert_offset;
  if (e_global < 0 || e < 0 || e >= p.num_local) return;  // tail block / expert of another shard

  if (tid < BM) sid_lds[tid] = sid_mine;

  // source row of tile row r whose routing slot is sid (gated: the slot's token; pad slots read
  // a valid row)
  auto src_row_of = [&](int sid, int r) -> int {
    if (GATED) return min(sid / p.topk, p.num_tokens - 1);
    return row0 + r;
  };

  // ---- direct-to-LDS staging: instruction = 8 rows x 128 bytes, lane -> (row, physical piece)
  uint32_t w_voff[4], x_voff[2];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int r = 32 * w + 8 * q + drow;  // tile-local weight row
    int n;
    if (GATED) n = (r < 128) ? nt * 128 + r : p.I + nt * 128 + (r - 128);
    else n = nt * 256 + r;
    n = min(n, p.N - 1);
    const int lc = dpc ^ ((r >> 1) & 7);  // logical piece that lands in physical piece dpc
    if (p.w_layout)
      w_voff[q] = (uint32_t)(n >> 4) * (uint32_t)KC * 2048u + (uint32_t)(lc >> 2) * 1024u +
                  (uint32_t)(((lc & 3) * 16 + (n & 15)) * 16);
    else
      w_voff[q] = (uint32_t)n * (uint32_t)K + (uint32_t)lc * 16u;
  }
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int r = 16 * w + 8 * q + drow;
    const int lc = dpc ^ ((r >> 1) & 7);
    x_voff[q] = (uint32_t)src_row_of(sid_x[q], r) * (uint32_t)K + (uint32_t)lc * 16u;
  }
  const unsigned char* wbase = p.w + (int64_t)e * p.N * K;
  const int w_kc_stride = p.w_layout ? 2048 : 128;
  // address = uniform base (scalar registers) + 32-bit lane offset: no 64-bit vector math
  const unsigned int w_dst0 = lds_addr(w_lds) + w * 4096, x_dst0 = lds_addr(x_lds) + w * 2048;
  auto issue_w = [&](int kc, int slot) {
    const uint32_t koff = (uint32_t)kc * (uint32_t)w_kc_stride;
    const unsigned int dst = w_dst0 + slot * kWSlot;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      dma16_global_to_lds(wbase, (uint32_t)(w_voff[q] + koff), dst + q * 1024);
  };
  auto issue_x = [&](int kc, int slot) {
    const uint32_t koff = (uint32_t)kc * 128u;
    const unsigned int dst = x_dst0 + slot * kXSlot;
#pragma unroll
    for (int q = 0; q < 2; ++q)
      dma16_global_to_lds(p.a, (uint32_t)(x_voff[q] + koff), dst + q * 1024);
  };
  // activation scales of chunks [kc0, kc0 + kSC) -> LDS (plain loads; 4 per thread)
  auto load_scales = [&](int kc0) {
    if (QT != 0) return;
    const int r = tid & (BM - 1), kq = tid >> 7;
    const float* sp = p.a_scale + (int64_t)src_row_of(sid_mine, r) * KC;
#pragma unroll
    for (int i = 0; i < kSC / 4; ++i) {
      const int kk = kq * (kSC / 4) + i;
      as_lds[kk][r] = sp[min(kc0 + kk, KC - 1)];
    }
    if (tid < 2 * kSC) {
      const int which = tid / kSC, kk = tid % kSC;
      const int blk = GATED ? (which ? (p.I >> 7) + nt : nt) : min(2 * nt + which, (p.N >> 7) - 1);
      ws_lds[which][kk] = p.w_scale[((int64_t)e * (p.N >> 7) + blk) * KC + min(kc0 + kk, KC - 1)];
    }
  };

  // ---- fragment reads (32x32 MFMA tiles).  Lane (j, h) takes, of row (tile row + j), the
  // logical 16-byte pieces 2q + h, q = 0..3 (chunk bytes 32 q + 16 h); piece lp of row r sits
  // in physical piece lp ^ ((r >> 1) & 7), and every tile starts at a multiple of 32 rows, so
  // the lane's four byte offsets are f0 ^ (32 q), the same for weights and activations.
  // Column tile ct of the wave starts at tile-local weight row
  //   gated: ct * 128 + cg * 32,   down: cg * 64 + ct * 32;   row tile rt at 64 rg + 32 rt.
  const int f0 = j * 128 + (((h ^ (j >> 1)) & 7) << 4);
  constexpr int kCtStride = GATED ? 128 * 128 : 32 * 128;  // bytes between the wave's column tiles
  int wf[4], xf[4];  // lane byte offsets inside a ring slot (column tile 0 / row tile 0)
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    wf[q] = (GATED ? cg * 32 : cg * 64) * 128 + (f0 ^ (q << 5));
    xf[q] = rg * (64 * 128) + (f0 ^ (q << 5));
  }
  const float* as_base = &as_lds[0][64 * rg + j];
  auto read_w = [&](int slot, int ct, u32x4 (&b)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      b[q] = *(const u32x4*)(w_lds + slot * kWSlot + ct * kCtStride + wf[q]);
  };
  auto read_x = [&](int slot, int kc, int rt, u32x4 (&x)[4], float& as) {
#pragma unroll
    for (int q = 0; q < 4; ++q) x[q] = *(const u32x4*)(x_lds + slot * kXSlot + rt * 4096 + xf[q]);
    as = QT == 0 ? as_base[(kc & (kSC - 1)) * BM + 32 * rt] : 1.0f;
  };

  // ---- weight block scales: wave-uniform, one per (128-column block, chunk), read from LDS
  // (gated: column tile 0 = gate block, 1 = up block; down: the wave's own 128-column block)
  const float* ws_row0 = ws_lds[GATED ? 0 : (cg >> 1)];
  const float* ws_row1 = ws_lds[GATED ? 1 : (cg >> 1)];

  f32x16 acc[2][2];  // [row tile][column tile]
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][ct][r] = 0.0f;
  f32x16 pp;
#pragma unroll
  for (int r = 0; r < 16; ++r) pp[r] = 0.0f;
  float psc = 0.0f;

  u32x4 ba[4], bb[4];  // weight fragments of column tile 0 / 1
  u32x4 x0[4], x1[4];  // activation fragments of row tile 0 / 1
  float as0 = 1.0f, as1 = 1.0f;
  float wsc[2] = {1.0f, 1.0f}, wsn[2] = {1.0f, 1.0f};

  // prologue: chunks 0..2 of the weights and 0..1 of the activations in flight, then the scales
  // (plain loads: issued after the copies so that they do not hold the copies back; the wait the
  // compiler puts before their LDS stores also covers every copy, which is older)
  issue_x(0, 0);
  issue_w(0, 0);
  if (KC > 1) {
    issue_x(1, 1);
    issue_w(1, 1);
  }
  if (KC > 2) issue_w(2, 2);
  load_scales(0);
  if (QT != 0) {
    if (KC > 2) __builtin_amdgcn_s_waitcnt(0x0F70 | 10);  // vmcnt(10): chunk 0 landed
    else __builtin_amdgcn_s_waitcnt(0x0F70);              // vmcnt(0)
  }
  __syncthreads();
  read_w(0, 0, ba);
  read_x(0, 0, 0, x0, as0);
  if (QT == 0) {
    wsc[0] = ws_row0[0];
    wsc[1] = ws_row1[0];
  }

  // one (row tile, column tile) step: two MFMAs over the chunk's two 64-byte halves, each
  // followed by half of the FMAs that retire the previous step's product into `prev`
  auto step = [&](const u32x4 (&b)[4], const u32x4 (&x)[4], f32x16& own, f32x16& prev, float sc) {
    if constexpr (QT == 0) {
      (void)own;
      f32x16 pc;
#pragma unroll
      for (int r = 0; r < 16; ++r) pc[r] = 0.0f;
      pc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cat8(b[0], b[1]), cat8(x[0], x[1]), pc, 0,
                                                           0, 0, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 8; ++r) prev[r] += pp[r] * psc;
      // keep the retiring FMAs inside this step (they would otherwise be sunk past the
      // following steps and run as one block with no MFMA to overlap)
      asm volatile("" : "+v"(prev));
      pc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cat8(b[2], b[3]), cat8(x[2], x[3]), pc, 0,
                                                           0, 0, 0, 0, 0);
#pragma unroll
      for (int r = 8; r < 16; ++r) prev[r] += pp[r] * psc;
      asm volatile("" : "+v"(prev));
      pp = pc;
      psc = sc;
    } else {
      (void)prev;
      (void)sc;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if constexpr (DT == DLB_DTYPE_BF16)
          own = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[q]),
                                                        __builtin_bit_cast(bf16x8, x[q]), own, 0, 0, 0);
        else
          own = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b[q]),
                                                       __builtin_bit_cast(f16x8, x[q]), own, 0, 0, 0);
      }
    }
  };
  // ring positions as scalars rotated once per chunk (no modulo in the loop): slot of chunk
  // kc (x_cur / w_cur), kc + 1 (x_nxt / w_nxt) and the one to refill (x_tgt: chunk kc + 2;
  // the weights of chunk kc + 3 go where chunk kc was)
  int x_cur = 0, x_nxt = 1, x_tgt = 2;
  int w_cur = 0, w_nxt = 1, w_aft = 2;
  // Chunk kc, steps in the order (ct 0, rt 0), (ct 0, rt 1), barrier, (ct 1, rt 0), (ct 1, rt 1).
  // On entry ba = W(kc, ct 0) and x0 = X(kc, rt 0) are in registers; bb and x1 are fetched
  // during step 0, the next chunk's ba during step 2 and x0 during step 3 (each register set
  // is free by then and the data landed with the barrier), so every LDS read has at least a
  // step of MFMAs to hide behind.
  for (int kc = 0; kc < KC; ++kc) {
    const bool more = kc + 1 < KC;
    read_w(w_cur, 1, bb);
    read_x(x_cur, kc, 1, x1, as1);
    __builtin_amdgcn_sched_barrier(0);
    step(ba, x0, acc[0][0], acc[1][1], as0 * wsc[0]);
    __builtin_amdgcn_sched_barrier(0);
    step(ba, x1, acc[1][0], acc[0][0], as1 * wsc[0]);
    __builtin_amdgcn_sched_barrier(0);
    if (more) {
      // chunk kc + 1 has landed once every wave's own loads of it are back
      if (kc + 2 < KC) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);  // W(kc + 2) may still fly
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (QT == 0 && ((kc + 1) & (kSC - 1)) == 0) {
        // rare (K > 2048 bytes): next tile of activation scales; every wave has fetched its
        // scales of chunk kc before the barrier above
        load_scales(kc + 1);
        __syncthreads();
      }
      if (kc + 2 < KC) issue_x(kc + 2, x_tgt);
      read_w(w_nxt, 0, ba);
      if (QT == 0) {
        wsn[0] = ws_row0[(kc + 1) & (kSC - 1)];
        wsn[1] = ws_row1[(kc + 1) & (kSC - 1)];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    step(bb, x0, acc[0][1], acc[1][0], as0 * wsc[1]);
    __builtin_amdgcn_sched_barrier(0);
    // the weights of chunk kc + 3 (least urgent) go out a step after the activations, which
    // spreads the workgroup's requests; still issued after X(kc + 2), as the waits assume
    if (kc + 3 < KC) issue_w(kc + 3, w_cur);
    if (more) read_x(x_nxt, kc + 1, 0, x0, as0);
    __builtin_amdgcn_sched_barrier(0);
    step(bb, x1, acc[1][1], acc[0][1], as1 * wsc[1]);
    __builtin_amdgcn_sched_barrier(0);
    {
      wsc[0] = wsn[0];
      wsc[1] = wsn[1];
      const int xr = x_cur;
      x_cur = x_nxt;
      x_nxt = x_tgt;
      x_tgt = xr;
      const int wr = w_cur;
      w_cur = w_nxt;
      w_nxt = w_aft;
      w_aft = wr;
    }
  }
  if constexpr (QT == 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[1][1][r] += pp[r] * psc;
  }

  // ---- epilogues: lane holds slot row (64 rg + 32 rt + j), columns (tile ct) + 8 (r / 4) +
  // 4 h + r % 4; a swap between the lane halves gives each lane 8 adjacent columns.
  // The output tile is assembled in LDS (the weight ring is free once every wave has left the
  // main loop) and written out as whole rows: 16-byte pieces, a row's pieces on adjacent lanes.
  const int rbase = 64 * rg;
  unsigned char* stage = w_lds;
  // copy `rows` x `row_bytes` from the staging tile to global rows given by dst_of(r) (nullptr: skip)
  auto flush_rows = [&](int row_bytes, auto dst_of) {
    const int ppr = row_bytes >> 4;            // 16-byte pieces per row
    const int total = BM * ppr;
    for (int u = tid; u < total; u += 512) {
      const int r = u / ppr, pc = u - r * ppr;
      unsigned char* dst = dst_of(r);
      if (dst) *(u32x4*)(dst + 16 * pc) = *(const u32x4*)(stage + r * row_bytes + 16 * pc);
    }
  };
  if (GATED && QT == 1) {
    // rounding points of the reference pipeline (fused_moe.py:166,351-352)
    __syncthreads();  // all waves are done with the rings
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      unsigned short* dst = (unsigned short*)stage + (rbase + 32 * rt + j) * 128 + cg * 32 + 8 * h;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        unsigned int o[2][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          float v[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r = 4 * (2 * pr + s) + i;
            const unsigned int gu = Elem<DT>::pack(acc[rt][0][r], acc[rt][1][r]);
            const float gate = Elem<DT>::lo(gu), up = Elem<DT>::hi(gu);
            const float sg = Elem<DT>::lo(Elem<DT>::pack(gate / (1.0f + __expf(-gate)), 0.0f));
            v[i] = sg * up;
          }
          o[s][0] = Elem<DT>::pack(v[0], v[1]);
          o[s][1] = Elem<DT>::pack(v[2], v[3]);
        }
        swap_halves(o[0][0], o[1][0]);
        swap_halves(o[0][1], o[1][1]);
        *(u32x4*)(dst + 16 * pr) = u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
      }
    }
    __syncthreads();
    flush_rows(256, [&](int r) -> unsigned char* {
      return p.hq + ((int64_t)(row0 + r) * p.I + nt * 128) * 2;
    });
  } else if (GATED) {
    float hv[2][16];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      float amax = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float gate = acc[rt][0][r];
        const float up = acc[rt][1][r];
        const float v = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;  // 1-ulp reciprocal
        hv[rt][r] = v;
        amax = fmaxf(amax, fabsf(v));
      }
      amax = max_xor32(amax);
      if (h == 0) red_lds[cg][rbase + 32 * rt + j] = amax;
    }
    __syncthreads();  // row maxima visible; all waves are done with the rings
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int r = rbase + 32 * rt + j;
      const float m = fmaxf(fmaxf(red_lds[0][r], red_lds[1][r]), fmaxf(red_lds[2][r], red_lds[3][r]));
      const float scale = fmaxf(m, kQuantEps) / kFp8Max;
      const float inv = __builtin_amdgcn_rcpf(scale);  // the stored scale stays exact
      unsigned int q[4];
#pragma unroll
      for (int s = 0; s < 4; ++s)
        q[s] = pack4_fp8(hv[rt][4 * s] * inv, hv[rt][4 * s + 1] * inv, hv[rt][4 * s + 2] * inv,
                         hv[rt][4 * s + 3] * inv);
      swap_halves(q[0], q[1]);
      swap_halves(q[2], q[3]);
      unsigned char* dst = stage + r * 128 + cg * 32 + 8 * h;
      *(u32x2*)(dst) = u32x2{q[0], q[1]};
      *(u32x2*)(dst + 16) = u32x2{q[2], q[3]};
      if (cg == 0 && h == 0) p.hs[(int64_t)(row0 + r) * (p.I >> 7) + nt] = scale;
    }
    __syncthreads();
    flush_rows(128, [&](int r) -> unsigned char* {
      return p.hq + (int64_t)(row0 + r) * p.I + nt * 128;
    });
  } else {
    __syncthreads();  // all waves are done with the rings (and sid_lds is long visible)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const int r = rbase + 32 * rt + j;
      const int sid = sid_lds[r];
      const float rw = sid < p.numel ? p.topk_w[sid] : 0.0f;
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) {
        unsigned short* dst = (unsigned short*)stage + r * 256 + cg * 64 + ct * 32 + 8 * h;
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
          unsigned int o[2][2];
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const int a = 4 * (2 * pr + s);
            o[s][0] = Elem<DT>::pack(acc[rt][ct][a] * rw, acc[rt][ct][a + 1] * rw);
            o[s][1] = Elem<DT>::pack(acc[rt][ct][a + 2] * rw, acc[rt][ct][a + 3] * rw);
          }
          swap_halves(o[0][0], o[1][0]);
          swap_halves(o[0][1], o[1][1]);
          *(u32x4*)(dst + 16 * pr) = u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
        }
      }
    }
    __syncthreads();
    const int ncols = min(256, p.N - nt * 256);  // multiple of 128
    const int ppr = ncols >> 3;                  // 16-byte pieces of a row that exist
    for (int u = tid; u < BM * 32; u += 512) {
      const int r = u >> 5, pc = u & 31;
      const int sid = sid_lds[r];
      if (sid < p.numel && pc < ppr)
        *(u32x4*)((unsigned short*)p.out + (int64_t)sid * p.N + nt * 256 + 8 * pc) =
            *(const u32x4*)(stage + r * 512 + 16 * pc);
    }
  }
}

// Same tile walk as moe_gemm_fp8_kernel (XCD x owns a contiguous range of the logical order).
template <bool GATED, int DT, int QT>
__global__ __launch_bounds__(512, 1) void moe_gemm_wide_kernel(const MoeGemmParams p) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int per_xcd = (p.grid_real + 7) >> 3;
  for (int i = slot; i < per_xcd; i += slots) {
    const int logical = xcd * per_xcd + i;
    if (logical < p.grid_real) moe_gemm_wide_tile<GATED, DT, QT>(p, logical);
    __syncthreads();  // the tile's LDS is reused by the next one
  }
}

// out[t, n] = sum_j in[t * topk + j, n], fp32 accumulation in slot order, one rounding
template <int DT>
__global__ __launch_bounds__(256) void moe_topk_sum_kernel(const u32x4* __restrict__ in,
                                                           u32x4* __restrict__ out,
                                                           int64_t total_vec, int vec_per_row,
                                                           int topk) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total_vec) return;
  const int64_t t = i / vec_per_row;
  const int col = (int)(i - t * vec_per_row);
  float s[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) s[q] = 0.0f;
  for (int j = 0; j < topk; ++j) {
    const u32x4 v = __builtin_nontemporal_load(in + (t * topk + j) * vec_per_row + col);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      s[2 * w] += Elem<DT>::lo(v[w]);
      s[2 * w + 1] += Elem<DT>::hi(v[w]);
    }
  }
  u32x4 r;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = Elem<DT>::pack(s[2 * w], s[2 * w + 1]);
  out[i] = r;
}

}  // namespace
}  // namespace dlb


extern "C" int dlb_per_token_group_quant_fp8(const void* x, void* xq, float* xs, int64_t M,
                                             int K, int64_t ld_x, int64_t ld_q, int64_t ld_s,
                                             int dtype, void* stream) {
  using namespace dlb;
  if (M < 0 || K < 0 || ld_x < K || ld_q < K || ld_s < K / 128) return DLB_ERR_BAD_ARG;
  if (M == 0 || K == 0) return DLB_OK;
  if (!x || !xq || !xs) return DLB_ERR_BAD_ARG;
  if (K % 128 != 0 || ld_x % 8 != 0 || ld_q % 8 != 0 || !aligned16(x) ||
      (reinterpret_cast<uintptr_t>(xq) & 7u) != 0)
    return DLB_ERR_UNSUPPORTED;
  const int gpr = K / 128;
  const int64_t total = M * gpr;
  const dim3 grid((uint32_t)ceil_div(total, 16 * kQuantUnroll));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DLB_DTYPE_BF16)
    hipLaunchKernelGGL(quant_fp8_group128_kernel<DLB_DTYPE_BF16>, grid, dim3(256), 0, s,
                       (const unsigned short*)x, (unsigned char*)xq, xs, total, gpr, ld_x, ld_q,
                       ld_s);
  else if (dtype == DLB_DTYPE_F16)
    hipLaunchKernelGGL(quant_fp8_group128_kernel<DLB_DTYPE_F16>, grid, dim3(256), 0, s,
                       (const unsigned short*)x, (unsigned char*)xq, xs, total, gpr, ld_x, ld_q,
                       ld_s);
  else
    return DLB_ERR_UNSUPPORTED;
  return launch_status();
}

namespace dlb {
namespace {

// resident workgroups of the 64-row kernel: two per CU, a multiple of the 8 XCDs
int persistent_workgroups() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    n = (cus * DLB_MOE_OCC) / 8 * 8;
    if (n < 8) n = 8;
  }
  return n;
}

template <bool GATED, int QT>
int launch_moe_gemm(const MoeGemmParams& p, int dtype, int block_m, hipStream_t s) {
  const uint32_t grid = (uint32_t)(ceil_div(p.grid_real, 8) * 8);
  // the 128-row kernel stores whole 16-byte pieces and addresses activation rows with 32 bits
  if (block_m == 128) {
    if ((p.hq && !aligned16(p.hq)) || (p.out && !aligned16(p.out))) return DLB_ERR_UNSUPPORTED;
    const int64_t a_rows = GATED ? p.num_tokens : (int64_t)p.num_mblocks * 128;
    if (a_rows * p.K >= (int64_t)0xffffffffu) return DLB_ERR_UNSUPPORTED;
  }
  // measured: one workgroup per tile (the dispatcher hands out tiles as slots free up) beats
  // resident workgroups walking a fixed share of the tiles, by 10 % for the gated GEMM and 3 %
  // for the down GEMM: blocks past the routed rows end at once and would unbalance fixed shares
  const uint32_t resident = (uint32_t)persistent_workgroups();
  const uint32_t pgrid = grid;
#define DLB_LAUNCH_GEMM(DT_)                                                                      \
  do {                                                                                          \
    if (p.w_layout)                                                                             \
      hipLaunchKernelGGL((moe_gemm_fp8_kernel<GATED, DT_, QT, 1>), dim3(pgrid), dim3(256), 0, s, p); \
    else                                                                                        \
      hipLaunchKernelGGL((moe_gemm_fp8_kernel<GATED, DT_, QT, 0>), dim3(pgrid), dim3(256), 0, s, p); \
  } while (0)
  const uint32_t wgrid = grid < resident / 2 ? grid : resident / 2;  // one 8-wave workgroup per CU
#define DLB_LAUNCH_WIDE(DT_) \
  hipLaunchKernelGGL((moe_gemm_wide_kernel<GATED, DT_, QT>), dim3(wgrid), dim3(512), 0, s, p)
  if (dtype == DLB_DTYPE_BF16) {
    if (block_m == 128) DLB_LAUNCH_WIDE(DLB_DTYPE_BF16);
    else DLB_LAUNCH_GEMM(DLB_DTYPE_BF16);
  } else if (dtype == DLB_DTYPE_F16) {
    if (block_m == 128) DLB_LAUNCH_WIDE(DLB_DTYPE_F16);
    else DLB_LAUNCH_GEMM(DLB_DTYPE_F16);
  } else {
    return DLB_ERR_UNSUPPORTED;
  }
#undef DLB_LAUNCH_GEMM
#undef DLB_LAUNCH_WIDE
  return launch_status();
}

// shared argument checks and parameter block of the four grouped-GEMM entry points;
// elem = bytes per operand element (1 for fp8, 2 for bf16/f16)
int fill_gemm_params(MoeGemmParams& p, bool gated, int elem, const void* a, const float* a_scale,
                     const void* w, const float* w_scale, const int32_t* sorted_ids,
                     const int32_t* expert_ids, int num_mblocks, int block_m, int num_tokens,
                     int topk, int H, int I, int expert_offset, int num_local_experts,
                     int w_layout) {
  const int Kel = gated ? H : I;       // reduction length (elements)
  const int N = gated ? 2 * I : H;     // weight rows per expert
  if (num_mblocks < 0 || H < 1 || I < 1) return DLB_ERR_BAD_ARG;
  if (num_mblocks == 0) return DLB_OK;
  if (!a || !w || !sorted_ids || !expert_ids) return DLB_ERR_BAD_ARG;
  if (elem == 1 && (!a_scale || !w_scale)) return DLB_ERR_BAD_ARG;
  if (num_tokens < 1 || topk < 1 || num_local_experts < 1) return DLB_ERR_BAD_ARG;
  if (block_m != 64 && block_m != 128) return DLB_ERR_UNSUPPORTED;
  // a row must be a whole number of 128-byte chunks; output tiles are 128 columns wide
  if ((Kel * elem) % 128 != 0 || I % 128 != 0 || H % 128 != 0) return DLB_ERR_UNSUPPORTED;
  if (!aligned16(a) || !aligned16(w)) return DLB_ERR_UNSUPPORTED;
  if ((int64_t)N * Kel * elem >= (int64_t)0xffffffffu) return DLB_ERR_UNSUPPORTED;  // 32-bit lane offsets
  p = MoeGemmParams{};
  p.a = (const unsigned char*)a;
  p.a_scale = a_scale;
  p.w = (const unsigned char*)w;
  p.w_scale = w_scale;
  p.sorted_ids = sorted_ids;
  p.expert_ids = expert_ids;
  p.num_mblocks = num_mblocks;
  p.num_ntiles = gated ? I / 128 : (int)ceil_div(H, 256);
  p.K = Kel * elem;
  p.N = N;
  p.KC = p.K / 128;
  p.topk = topk;
  p.numel = num_tokens * topk;
  p.num_tokens = num_tokens;
  p.expert_offset = expert_offset;
  p.num_local = num_local_experts;
  p.w_layout = w_layout ? 1 : 0;
  p.I = I;
  p.grid_real = p.num_mblocks * p.num_ntiles;
  return DLB_OK;
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_moe_gemm_fp8_gate_up(const void* xq, const float* xs, const void* w1q,
                                        const float* w1s, const int32_t* sorted_ids,
                                        const int32_t* expert_ids, int num_mblocks, int block_m,
                                        int num_tokens, int topk, int H, int I,
                                        int expert_offset, int num_local_experts, int w_layout,
                                        void* hq, float* hs, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, true, 1, xq, xs, w1q, w1s, sorted_ids, expert_ids,
                                  num_mblocks, block_m, num_tokens, topk, H, I, expert_offset,
                                  num_local_experts, w_layout);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!hq || !hs) return DLB_ERR_BAD_ARG;
  if (!aligned16(hq)) return DLB_ERR_UNSUPPORTED;
  p.hq = (unsigned char*)hq;
  p.hs = hs;
  return launch_moe_gemm<true, 0>(p, DLB_DTYPE_BF16, block_m, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_fp8_down(const void* hq, const float* hs, const void* w2q,
                                     const float* w2s, const int32_t* sorted_ids,
                                     const int32_t* expert_ids, const float* topk_weights,
                                     int num_mblocks, int block_m, int num_tokens, int topk,
                                     int H, int I, int expert_offset, int num_local_experts,
                                     int w_layout, void* out, int out_dtype, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, false, 1, hq, hs, w2q, w2s, sorted_ids, expert_ids,
                                  num_mblocks, block_m, num_tokens, topk, H, I, expert_offset,
                                  num_local_experts, w_layout);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!out || !topk_weights) return DLB_ERR_BAD_ARG;
  if (!aligned16(out)) return DLB_ERR_UNSUPPORTED;
  p.out = out;
  p.topk_w = topk_weights;
  return launch_moe_gemm<false, 0>(p, out_dtype, block_m, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_16bit_gate_up(const void* x, const void* w1,
                                          const int32_t* sorted_ids, const int32_t* expert_ids,
                                          int num_mblocks, int block_m, int num_tokens, int topk,
                                          int H, int I, int expert_offset, int num_local_experts,
                                          int w_layout, void* act, int dtype, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, true, 2, x, nullptr, w1, nullptr, sorted_ids, expert_ids,
                                  num_mblocks, block_m, num_tokens, topk, H, I, expert_offset,
                                  num_local_experts, w_layout);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!act) return DLB_ERR_BAD_ARG;
  if (!aligned16(act)) return DLB_ERR_UNSUPPORTED;
  p.hq = (unsigned char*)act;
  return launch_moe_gemm<true, 1>(p, dtype, block_m, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_16bit_down(const void* act, const void* w2,
                                       const int32_t* sorted_ids, const int32_t* expert_ids,
                                       const float* topk_weights, int num_mblocks, int block_m,
                                       int num_tokens, int topk, int H, int I, int expert_offset,
                                       int num_local_experts, int w_layout, void* out, int dtype,
                                       void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, false, 2, act, nullptr, w2, nullptr, sorted_ids, expert_ids,
                                  num_mblocks, block_m, num_tokens, topk, H, I, expert_offset,
                                  num_local_experts, w_layout);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!out || !topk_weights) return DLB_ERR_BAD_ARG;
  if (!aligned16(out)) return DLB_ERR_UNSUPPORTED;
  p.out = out;
  p.topk_w = topk_weights;
  return launch_moe_gemm<false, 1>(p, dtype, block_m, (hipStream_t)stream);
}

extern "C" int dlb_moe_topk_sum(const void* in, void* out, int64_t num_tokens, int topk,
                                int64_t N, int dtype, void* stream) {
  using namespace dlb;
  if (num_tokens < 0 || topk < 1 || N < 0) return DLB_ERR_BAD_ARG;
  if (num_tokens == 0 || N == 0) return DLB_OK;
  if (!in || !out) return DLB_ERR_BAD_ARG;
  if (N % 8 != 0 || !aligned16(in) || !aligned16(out)) return DLB_ERR_UNSUPPORTED;
  const int64_t total = num_tokens * (N / 8);
  const dim3 grid((uint32_t)ceil_div(total, 256));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DLB_DTYPE_BF16)
    hipLaunchKernelGGL(moe_topk_sum_kernel<DLB_DTYPE_BF16>, grid, dim3(256), 0, s,
                       (const u32x4*)in, (u32x4*)out, total, (int)(N / 8), topk);
  else if (dtype == DLB_DTYPE_F16)
    hipLaunchKernelGGL(moe_topk_sum_kernel<DLB_DTYPE_F16>, grid, dim3(256), 0, s,
                       (const u32x4*)in, (u32x4*)out, total, (int)(N / 8), topk);
  else
    return DLB_ERR_UNSUPPORTED;
  return launch_status();
}
