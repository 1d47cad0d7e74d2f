// fp8 (OCP e4m3fn) fused-MoE building blocks for gfx950:
//   * per-token-group activation quantisation (groups of 128 along K, fp32 scales);
//   * expert-grouped GEMM over block-aligned routing (64-row blocks, one expert per block) on
//     the 16x16x128 f8f6f4 MFMA, with the block scales applied per 128-deep K chunk:
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
// The same kernel also runs unquantised bf16/f16 operands (QT = 1): the reference's own
// fused_moe, with 16x16x32 MFMAs accumulating in place and no scales.
//
// GEMM mapping.  The MFMA runs "transposed": weight rows are the A operand (M index = output
// column n), activations the B operand (N index = token row), so a lane's four accumulator
// registers are four consecutive n of ONE token: the activation scale is a per-lane scalar
// and the epilogues store 4 adjacent outputs.  Weight fragments go straight from HBM/L2 into
// operand registers (each wave owns its own n range, so nothing is shared between waves);
// only the 64 x 128-byte activation chunk is staged through LDS, double-buffered.
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


__device__ __forceinline__ f32x4 mfma_fp8(const i32x8& a, const i32x8& b) {
  const f32x4 z = {0.f, 0.f, 0.f, 0.f};
  // cbsz = blgp = 0: both operands e4m3; zero scale operands select the unscaled opcode
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, z, 0, 0, 0, 0, 0, 0);
}

template <int DT>
__device__ __forceinline__ f32x4 mfma_16bit(const i32x8& a, const i32x8& b, f32x4 c) {
  // one 128-byte chunk = 64 elements = two 16x16x32 steps on the two operand halves
  typedef __attribute__((ext_vector_type(4))) int i32x4;
  const i32x4 a0 = {a[0], a[1], a[2], a[3]}, a1 = {a[4], a[5], a[6], a[7]};
  const i32x4 b0 = {b[0], b[1], b[2], b[3]}, b1 = {b[4], b[5], b[6], b[7]};
  if constexpr (DT == DLB_DTYPE_BF16) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a0),
                                                __builtin_bit_cast(bf16x8, b0), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a1),
                                                __builtin_bit_cast(bf16x8, b1), c, 0, 0, 0);
  } else {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a0),
                                               __builtin_bit_cast(f16x8, b0), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a1),
                                               __builtin_bit_cast(f16x8, b1), c, 0, 0, 0);
  }
  return c;
}

// QT = 0: fp8 operands with block scales; QT = 1: 16-bit operands of type DT, no scales.
// GATED = true : gate_up GEMM (N = 2I), tile = 128 gate cols + the matching 128 up cols,
//                epilogue silu(gate) * up -> fp8 + per-128 scale, rows kept in sorted order.
// GATED = false: down GEMM, tile = 256 cols, epilogue * routing weight -> out[slot, n].
// BM = rows (routing slots) per workgroup = the alignment block of the routing (64 or 128).
#ifndef DLB_MOE_OCC
#define DLB_MOE_OCC 2
#endif
template <bool GATED, int DT, int BM, int QT>
__device__ __forceinline__ void moe_gemm_fp8_tile(const MoeGemmParams& p, const int logical) {
  constexpr int kBM = BM;
  constexpr int MT = BM / 16;          // 16-token sub-tiles
  constexpr int SKC = 2;               // 128-byte K chunks per activation stage
#ifndef DLB_MOE_PD
#define DLB_MOE_PD 2
#endif
  constexpr int PD = DLB_MOE_PD;       // weight-fragment ring depth (chunks in flight + 1)
  constexpr int TPR = 256 / BM;        // staging threads per activation row
  constexpr int AU = SKC * 8 / TPR;    // 16-byte units per staging thread and stage
  constexpr int kARow = SKC * 128 + 16;  // LDS row pitch of an activation stage (bytes)
  static_assert(SKC <= TPR, "one staging thread per (row, chunk) loads the scale");
  __shared__ __attribute__((aligned(16))) unsigned char a_lds[2][kBM * kARow];
  __shared__ __attribute__((aligned(16))) float as_lds[2][SKC][kBM];
  __shared__ float red_lds[4][kBM];
  __shared__ int32_t sid_lds[kBM];

  const int mb = logical % p.num_mblocks;
  const int nt = logical / p.num_mblocks;
  const int e_global = p.expert_ids[mb];
  const int e = e_global - p.expert_offset;
  if (e_global < 0 || e < 0 || e >= p.num_local) return;  // tail block / expert of another shard

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int row0 = mb * kBM;
  const int K = p.K, KC = p.KC;

  if (tid < kBM) sid_lds[tid] = p.sorted_ids[row0 + tid];
  static_assert(BM == 64 || BM == 128, "BM");
  static_assert(AU == SKC * (BM / 32), "staging units per thread");

  // ---- activation chunk staging.  Data: 8 consecutive lanes fetch one row's 128-byte chunk
  // (a full cache line per row and instruction), 32 rows per pass, BM / 32 passes per chunk.
  // Scales: thread (row = tid / TPR, chunk = tid % TPR < SKC) fetches one float per stage.
  constexpr int RP = BM / 32;            // row passes per chunk
  const int arow = tid / TPR, aseg = tid % TPR;
  const int prow = tid >> 3, piece = tid & 7;
  const unsigned char* a_ptr[RP];
  const float* as_ptr;
  {
    auto src_row_of = [&](int r) -> int64_t {
      if (GATED) {
        const int sid = p.sorted_ids[row0 + r];
        return min(sid / p.topk, p.num_tokens - 1);  // pad slots read a valid row
      }
      return row0 + r;
    };
#pragma unroll
    for (int k = 0; k < RP; ++k) a_ptr[k] = p.a + src_row_of(32 * k + prow) * K + 16 * piece;
    as_ptr = QT == 0 ? p.a_scale + src_row_of(arow) * KC : nullptr;
  }

  // ---- weight fragments: sub-tile j of this wave covers 16 output columns
  int ncol[4];   // first column of sub-tile j in the expert's [N, K] matrix
  int sblk[4];   // its 128-row scale block
  if (GATED) {
    const int n0 = nt * 128 + wave * 32;
    ncol[0] = n0;
    ncol[1] = n0 + 16;
    ncol[2] = p.I + n0;
    ncol[3] = p.I + n0 + 16;
  } else {
    const int n0 = nt * 256 + wave * 64;
#pragma unroll
    for (int j = 0; j < 4; ++j) ncol[j] = n0 + 16 * j;
  }
  // Weight addressing: one wave-uniform base per expert (kept in scalar registers) plus a
  // 32-bit per-lane byte offset per sub-tile; the block scales of a sub-tile are wave-uniform
  // and come through scalar loads.
  const unsigned char* wbase = p.w + (int64_t)e * p.N * K;
  uint32_t woff[4];
  const float* ws_ptr[4];
  // byte distance between consecutive K chunks / between the two 16-byte operand halves
  const int w_kc_stride = p.w_layout ? 2048 : 128;
  const int w_hi_off = p.w_layout ? 1024 : 64;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    sblk[j] = __builtin_amdgcn_readfirstlane(min(ncol[j] >> 7, (p.N >> 7) - 1));
    if (p.w_layout) {
      // operand-order storage: per (16-row tile, chunk) one 2 KB block = [half][lane][16 B],
      // so each of the two loads of a fragment is one contiguous 1 KB wave access
      const int nb = min(ncol[j] >> 4, (p.N >> 4) - 1);
      woff[j] = (uint32_t)nb * (uint32_t)KC * 2048u + (uint32_t)lane * 16u;
    } else {
      // row-major storage: lanes of group g take K bytes [16g, 16g+16) and [64+16g, 64+16g+16)
      const int n = min(ncol[j] + c, p.N - 1);
      woff[j] = (uint32_t)n * (uint32_t)K + 16u * g;
    }
    ws_ptr[j] = QT == 0 ? p.w_scale + ((int64_t)e * (p.N >> 7) + sblk[j]) * KC : nullptr;
  }

  f32x4 acc[MT][4];  // [token sub-tile mt][column sub-tile j]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[mt][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Pipeline: activations move global -> registers -> LDS in stages of SKC chunks, one stage
  // ahead, one barrier per stage; weight fragments sit in a ring of PD chunks, loaded PD-1
  // chunks ahead of their use; the scale-and-accumulate FMAs of one 16-token step are issued
  // between the MFMAs of the next step so the matrix pipe does not wait for the VALU.
  u32x4 areg[AU];
  float asreg = 0.0f;
  i32x8 breg[PD][4];
  // block scales of a wave's sub-tiles: sub-tiles 0,1 and 2,3 share a 128-column block (gate /
  // up columns; one block for all four in the down GEMM)
  constexpr int NSC = GATED ? 2 : 1;
  float bsreg[PD][NSC];
  const int NS = (KC + SKC - 1) / SKC;

  auto load_a = [&](int st) {  // stage st -> registers (chunks past K are clamped, unused)
    const int kc0 = st * SKC;
#pragma unroll
    for (int u = 0; u < AU; ++u) {
      const int kc = min(kc0 + u / RP, KC - 1);
      areg[u] = *(const u32x4*)(a_ptr[u % RP] + kc * 128);
    }
    if (QT == 0 && aseg < SKC) asreg = as_ptr[min(kc0 + aseg, KC - 1)];
  };
  auto store_a = [&](int buf) {
    unsigned char* dst = a_lds[buf] + prow * kARow + 16 * piece;
#pragma unroll
    for (int u = 0; u < AU; ++u) *(u32x4*)(dst + (u % RP) * 32 * kARow + (u / RP) * 128) = areg[u];
    if (QT == 0 && aseg < SKC) as_lds[buf][aseg][arow] = asreg;
  };
  auto load_b = [&](int kc, i32x8 (&b)[4], float (&bs)[NSC]) {
    if (kc >= KC) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned char* src = wbase + kc * w_kc_stride;
      const u32x4 lo = *(const u32x4*)(src + woff[j]);
      const u32x4 hi = *(const u32x4*)(src + w_hi_off + woff[j]);
      b[j] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                   (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    }
#pragma unroll
    for (int q = 0; q < NSC; ++q) bs[q] = QT == 0 ? ws_ptr[2 * q][kc] : 1.0f;
  };

  // software pipeline state: products of the previous 16-token step and their scales
  f32x4 pp[4];
  float psc[NSC];
#pragma unroll
  for (int j = 0; j < 4; ++j) pp[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int q = 0; q < NSC; ++q) psc[q] = 0.0f;
  // A stage is SKC * MT steps of 16 tokens x one chunk.  Step t issues its 4 MFMAs, each
  // followed by the FMAs that retire one product of step t - 1 (for the first step of a
  // stage: the last step of the previous stage); the activation fragment of step t + 1 is
  // fetched from LDS before the MFMAs of step t so its latency hides behind them.
  auto read_x = [&](int buf, int ci, int mt, i32x8& x, float& as) {
    const unsigned char* src = a_lds[buf] + (16 * mt + c) * kARow + ci * 128 + 16 * g;
    const u32x4 lo = *(const u32x4*)(src);
    const u32x4 hi = *(const u32x4*)(src + 64);
    x = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
              (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    as = QT == 0 ? as_lds[buf][ci][16 * mt + c] : 1.0f;
  };
  auto do_stage = [&](auto jtag, int st) {
    constexpr int J = decltype(jtag)::value;  // st % PD
    const int buf = st & 1;
    const int nchunks = min(SKC, KC - st * SKC);  // chunks of this stage that exist (uniform)
    i32x8 xq[2];
    float asq[2];
    read_x(buf, 0, 0, xq[0], asq[0]);
#pragma unroll
    for (int ci = 0; ci < SKC; ++ci) {
      // ring slot of chunk kc = st * SKC + ci is kc % PD, the slot being refilled holds
      // chunk kc + PD - 1; both are compile-time constants after unrolling
      constexpr int kBase = (J * SKC) % PD;
      const int slot = (kBase + ci) % PD;
      const int refill = (kBase + ci + PD - 1) % PD;
      if (ci < nchunks) {
        load_b(st * SKC + ci + PD - 1, breg[refill], bsreg[refill]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int t = ci * MT + mt;
          const int pm = (mt == 0) ? MT - 1 : mt - 1;
          // prefetch the next step's fragment (same stage only)
          if (mt + 1 < MT) {
            read_x(buf, ci, mt + 1, xq[(t + 1) & 1], asq[(t + 1) & 1]);
          } else if (ci + 1 < SKC) {
            if (ci + 1 < nchunks) read_x(buf, ci + 1, 0, xq[(t + 1) & 1], asq[(t + 1) & 1]);
          }
          if constexpr (QT == 0) {
            f32x4 pc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              pc[j] = mfma_fp8(breg[slot][j], xq[t & 1]);
              acc[pm][j] += pp[j] * psc[GATED ? (j >> 1) : 0];
            }
            // keep the retiring FMAs next to these MFMAs (the optimiser would otherwise sink
            // them into one long VALU run with nothing to overlap)
            asm volatile("" : "+v"(acc[pm][0]), "+v"(acc[pm][1]), "+v"(acc[pm][2]), "+v"(acc[pm][3]));
#pragma unroll
            for (int j = 0; j < 4; ++j) pp[j] = pc[j];
#pragma unroll
            for (int q = 0; q < NSC; ++q) psc[q] = asq[t & 1] * bsreg[slot][q];
          } else {
            (void)pm;
#pragma unroll
            for (int j = 0; j < 4; ++j)
              acc[mt][j] = mfma_16bit<DT>(breg[slot][j], xq[t & 1], acc[mt][j]);
          }
        }
      }
    }
    if (st + 1 < NS) store_a(buf ^ 1);   // stage st + 1 was loaded into registers a stage ago
    if (st + 2 < NS) load_a(st + 2);
    __syncthreads();
  };

  load_a(0);
#pragma unroll
  for (int t = 0; t < PD - 1; ++t) load_b(t, breg[t], bsreg[t]);
  store_a(0);
  if (NS > 1) load_a(1);
  __syncthreads();
  for (int st = 0; st < NS; st += PD) {
    do_stage(std::integral_constant<int, 0>{}, st);
    if (PD > 1 && st + 1 < NS) do_stage(std::integral_constant<int, 1 % PD>{}, st + 1);
    if (PD > 2 && st + 2 < NS) do_stage(std::integral_constant<int, 2 % PD>{}, st + 2);
  }
  // retire the products of the very last step
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[MT - 1][j] += pp[j] * psc[GATED ? (j >> 1) : 0];

  // ---- epilogues: lane holds token (16*mt + c), columns ncol[j] + 4*g + i
  if (GATED && QT == 1) {
    // rounding points of the reference pipeline (fused_moe.py:166,351-352): GEMM result,
    // silu(gate) and the product are each rounded to the activation type
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int64_t orow = row0 + 16 * mt + c;
      unsigned short* dst = (unsigned short*)p.hq + orow * p.I + nt * 128 + wave * 32 + 4 * g;
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned int gu = Elem<DT>::pack(acc[mt][jg][i], acc[mt][jg + 2][i]);
          const float gate = Elem<DT>::lo(gu), up = Elem<DT>::hi(gu);
          const float sg = Elem<DT>::lo(Elem<DT>::pack(gate / (1.0f + __expf(-gate)), 0.0f));
          v[i] = sg * up;
        }
        u32x2 o2;
        o2[0] = Elem<DT>::pack(v[0], v[1]);
        o2[1] = Elem<DT>::pack(v[2], v[3]);
        *(u32x2*)(dst + 16 * jg) = o2;
      }
    }
  } else if (GATED) {
    float h[MT][2][4];
    float amax[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      amax[mt] = 0.0f;
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float gate = acc[mt][jg][i];
          const float up = acc[mt][jg + 2][i];
          const float v = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;  // 1-ulp reciprocal
          h[mt][jg][i] = v;
          amax[mt] = fmaxf(amax[mt], fabsf(v));
        }
      }
      amax[mt] = fmaxf(amax[mt], __shfl_xor(amax[mt], 16));
      amax[mt] = fmaxf(amax[mt], __shfl_xor(amax[mt], 32));
      if (g == 0) red_lds[wave][16 * mt + c] = amax[mt];
    }
    __syncthreads();
    const int scol = nt;  // 128-column group index of the intermediate
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int r = 16 * mt + c;
      const float m = fmaxf(fmaxf(red_lds[0][r], red_lds[1][r]), fmaxf(red_lds[2][r], red_lds[3][r]));
      const float scale = fmaxf(m, kQuantEps) / kFp8Max;
      const float inv = __builtin_amdgcn_rcpf(scale);  // the stored scale stays exact
      const int64_t orow = row0 + r;
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
        const unsigned int q = pack4_fp8(h[mt][jg][0] * inv, h[mt][jg][1] * inv,
                                         h[mt][jg][2] * inv, h[mt][jg][3] * inv);
        *(unsigned int*)(p.hq + orow * p.I + nt * 128 + wave * 32 + 16 * jg + 4 * g) = q;
      }
      if (wave == 0 && g == 0) p.hs[orow * (p.I >> 7) + scol] = scale;
    }
  } else {
    __syncthreads();  // sid_lds visible (also true after the main loop's barriers)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int sid = sid_lds[16 * mt + c];
      if (sid < p.numel) {
        const float rw = p.topk_w[sid];
        unsigned short* orow = (unsigned short*)p.out + (int64_t)sid * p.N;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = ncol[j] + 4 * g;
          if (n < p.N) {
            u32x2 o2;
            o2[0] = Elem<DT>::pack(acc[mt][j][0] * rw, acc[mt][j][1] * rw);
            o2[1] = Elem<DT>::pack(acc[mt][j][2] * rw, acc[mt][j][3] * rw);
            *(u32x2*)(orow + n) = o2;
          }
        }
      }
    }
  }
}

// Workgroup ids are dealt round-robin to the 8 XCDs, so XCD x takes the contiguous range
// [x * per_xcd, (x + 1) * per_xcd) of the logical tile order (same column tile, consecutive
// row blocks = mostly the same expert: neighbours share an L2) and its workgroups take
// consecutive tiles of it.  With fewer workgroups than tiles (a resident launch, two per CU)
// every workgroup walks a fixed sequence of tiles; with one workgroup per tile the loop runs
// once.
template <bool GATED, int DT, int BM, int QT>
__global__ __launch_bounds__(256, DLB_MOE_OCC) void moe_gemm_fp8_kernel(const MoeGemmParams p) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
  const int per_xcd = (p.grid_real + 7) >> 3;
  for (int i = slot; i < per_xcd; i += slots) {
    const int logical = xcd * per_xcd + i;
    if (logical < p.grid_real) moe_gemm_fp8_tile<GATED, DT, BM, QT>(p, logical);
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
  constexpr int BM = 128, BN = 256, MT = 4;
  constexpr int kWSlot = BN * 128;  // bytes of one weight ring slot
  constexpr int kXSlot = BM * 128;  // bytes of one activation ring slot
  constexpr int kSC = 16;           // chunks of activation scales resident in LDS
  __shared__ __attribute__((aligned(1024))) unsigned char w_lds[3 * kWSlot];
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds[3 * kXSlot];
  __shared__ float as_lds[kSC][BM];
  __shared__ float ws_lds[2][kSC];  // block scales of the tile's two 128-column weight blocks
  __shared__ float red_lds[4][BM];
  __shared__ int32_t sid_lds[BM];

  const int mb = logical % p.num_mblocks;
  const int nt = logical / p.num_mblocks;
  const int e_global = p.expert_ids[mb];
  const int e = e_global - p.expert_offset;
  if (e_global < 0 || e < 0 || e >= p.num_local) return;  // tail block / expert of another shard

  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave id, kept in scalar registers
  const int lane = tid & 63;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int rg = w >> 2;  // waves w and w + 4 share a SIMD: give them different row groups
  const int cg = w & 3;
  const int row0 = mb * BM;
  const int K = p.K, KC = p.KC;

  if (tid < BM) sid_lds[tid] = p.sorted_ids[row0 + tid];

  auto src_row_of = [&](int r) -> int {
    if (GATED) {
      const int sid = p.sorted_ids[row0 + r];
      return min(sid / p.topk, p.num_tokens - 1);  // pad slots read a valid row
    }
    return row0 + r;
  };

  // ---- direct-to-LDS staging: instruction = 8 rows x 128 bytes, lane -> (row, physical piece)
  const int drow = lane >> 3, dpc = lane & 7;
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
    x_voff[q] = (uint32_t)src_row_of(r) * (uint32_t)K + (uint32_t)lc * 16u;
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
    const float* sp = p.a_scale + (int64_t)src_row_of(r) * KC;
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

  // ---- fragment reads: lane (c, g) takes pieces g and g + 4 of row (tile row + c)
  // Per lane one base pointer per operand and half; slot and tile offsets are a scalar add and
  // an immediate.  Column sub-tile j starts at tile-local weight row
  //   gated: (j >> 1) * 128 + cg * 32 + (j & 1) * 16,   down: cg * 64 + j * 16.
  const int lo_off = c * 128 + (((g) ^ (c >> 1)) & 7) * 16;
  const int hi_off = c * 128 + (((g + 4) ^ (c >> 1)) & 7) * 16;
  const int wcg = (GATED ? cg * 32 : cg * 64) * 128;
  const unsigned char* w_lo = w_lds + wcg + lo_off;
  const unsigned char* w_hi = w_lds + wcg + hi_off;
  const unsigned char* x_lo = x_lds + rg * (64 * 128) + lo_off;
  const unsigned char* x_hi = x_lds + rg * (64 * 128) + hi_off;
  const float* as_base = &as_lds[0][64 * rg + c];
  auto read_w = [&](int slot, i32x8 (&b)[4]) {
    const unsigned char* bl = w_lo + slot * kWSlot;
    const unsigned char* bh = w_hi + slot * kWSlot;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      constexpr int kUp = 128 * 128;  // gated: up rows follow the 128 gate rows
      const int off = GATED ? (j >> 1) * kUp + (j & 1) * 2048 : j * 2048;
      const u32x4 lo = *(const u32x4*)(bl + off);
      const u32x4 hi = *(const u32x4*)(bh + off);
      b[j] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                   (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    }
  };
  auto read_x = [&](int slot, int kc, int mt, i32x8& x, float& as) {
    const u32x4 lo = *(const u32x4*)(x_lo + slot * kXSlot + mt * 2048);
    const u32x4 hi = *(const u32x4*)(x_hi + slot * kXSlot + mt * 2048);
    x = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
              (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
    as = QT == 0 ? as_base[(kc & (kSC - 1)) * BM + 16 * mt] : 1.0f;
  };

  // ---- weight block scales: wave-uniform, one per (128-column block, chunk), read from LDS
  // (gated: block 0 = gate columns, 1 = up columns; down: the wave's own 128-column block)
  const float* ws_row0 = ws_lds[GATED ? 0 : (cg >> 1)];
  const float* ws_row1 = ws_lds[GATED ? 1 : (cg >> 1)];

  f32x4 acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[mt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 pp[4];
  float psc[2] = {0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) pp[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  i32x8 b0[4], b1[4];
  i32x8 xq[2];
  float asq[2];
  float wsc[2] = {1.0f, 1.0f}, wsn[2] = {1.0f, 1.0f};

  // prologue: scales, chunks 0..2 of the weights and 0..1 of the activations in flight
  load_scales(0);
  issue_x(0, 0);
  issue_w(0, 0);
  if (KC > 1) {
    issue_x(1, 1);
    issue_w(1, 1);
  }
  if (KC > 2) {
    issue_w(2, 2);
    __builtin_amdgcn_s_waitcnt(0x0F70 | 10);  // vmcnt(10): chunk 0 landed, 10 newer loads may fly
  } else {
    __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0)
  }
  __syncthreads();
  read_w(0, b0);
  read_x(0, 0, 0, xq[0], asq[0]);
  if (QT == 0) {
    wsc[0] = ws_row0[0];
    wsc[1] = ws_row1[0];
  }

  // one 16-row step: 4 MFMAs, each followed by the FMAs retiring one product of the previous step
  auto step = [&](const i32x8 (&b)[4], int mt, int cur) {
    const int pm = (mt == 0) ? MT - 1 : mt - 1;
    if constexpr (QT == 0) {
      f32x4 pc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pc[j] = mfma_fp8(b[j], xq[cur]);
        acc[pm][j] += pp[j] * psc[GATED ? (j >> 1) : 0];
      }
      // keep the retiring FMAs inside this step (they would otherwise be sunk past the
      // following steps and run as one block with no MFMA to overlap)
      asm volatile("" : "+v"(acc[pm][0]), "+v"(acc[pm][1]), "+v"(acc[pm][2]), "+v"(acc[pm][3]));
#pragma unroll
      for (int j = 0; j < 4; ++j) pp[j] = pc[j];
      psc[0] = asq[cur] * wsc[0];
      psc[1] = asq[cur] * wsc[1];
    } else {
      (void)pm;
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[mt][j] = mfma_16bit<DT>(b[j], xq[cur], acc[mt][j]);
    }
  };
  // ring positions as scalars rotated once per chunk (no modulo in the loop): slot of chunk
  // kc (x_cur / w_cur), kc + 1 (x_nxt / w_nxt) and the one to refill (x_tgt: chunk kc + 2;
  // the weights of chunk kc + 3 go where chunk kc was)
  int x_cur = 0, x_nxt = 1, x_tgt = 2;
  int w_cur = 0, w_nxt = 1, w_aft = 2;
  auto rotate = [&]() {
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
  };
  auto do_chunk = [&](const i32x8 (&bc)[4], i32x8 (&bn)[4], int kc) {
    const bool more = kc + 1 < KC;
    read_x(x_cur, kc, 1, xq[1], asq[1]);
    __builtin_amdgcn_sched_barrier(0);
    step(bc, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    read_x(x_cur, kc, 2, xq[0], asq[0]);
    __builtin_amdgcn_sched_barrier(0);
    step(bc, 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    if (more) {
      // chunk kc + 1 has landed once every wave's own loads of it are back
      if (kc + 2 < KC) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);  // W(kc + 2) may still fly
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      if (QT == 0 && ((kc + 1) & (kSC - 1)) == 0) {
        // rare (K > 2048 bytes): next tile of activation scales; every wave is past its reads
        // of the old tile once it has the step-3 fragment, so fetch that first
        read_x(x_cur, kc, 3, xq[1], asq[1]);
        __syncthreads();
        load_scales(kc + 1);
        __syncthreads();
      } else {
        __syncthreads();
        read_x(x_cur, kc, 3, xq[1], asq[1]);
      }
      if (kc + 2 < KC) issue_x(kc + 2, x_tgt);
      read_w(w_nxt, bn);
      if (QT == 0) {
        wsn[0] = ws_row0[(kc + 1) & (kSC - 1)];
        wsn[1] = ws_row1[(kc + 1) & (kSC - 1)];
      }
    } else {
      read_x(x_cur, kc, 3, xq[1], asq[1]);
    }
    __builtin_amdgcn_sched_barrier(0);
    step(bc, 2, 0);
    __builtin_amdgcn_sched_barrier(0);
    // the weights of chunk kc + 3 (least urgent) go out a step after the activations, which
    // spreads the workgroup's requests; still issued after X(kc + 2), as the waits assume
    if (kc + 3 < KC) issue_w(kc + 3, w_cur);
    if (more) read_x(x_nxt, kc + 1, 0, xq[0], asq[0]);
    __builtin_amdgcn_sched_barrier(0);
    step(bc, 3, 1);
    __builtin_amdgcn_sched_barrier(0);
    rotate();
  };
  for (int kc = 0; kc < KC; kc += 2) {
    do_chunk(b0, b1, kc);
    if (kc + 1 < KC) do_chunk(b1, b0, kc + 1);
  }
  if constexpr (QT == 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[MT - 1][j] += pp[j] * psc[GATED ? (j >> 1) : 0];
  }

  // ---- epilogues: lane holds slot row (64*rg + 16*mt + c), columns (sub-tile j) + 4*g + i.
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
    for (int mt = 0; mt < MT; ++mt) {
      unsigned short* dst = (unsigned short*)stage + (rbase + 16 * mt + c) * 128 + cg * 32 + 4 * g;
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned int gu = Elem<DT>::pack(acc[mt][jg][i], acc[mt][jg + 2][i]);
          const float gate = Elem<DT>::lo(gu), up = Elem<DT>::hi(gu);
          const float sg = Elem<DT>::lo(Elem<DT>::pack(gate / (1.0f + __expf(-gate)), 0.0f));
          v[i] = sg * up;
        }
        u32x2 o2;
        o2[0] = Elem<DT>::pack(v[0], v[1]);
        o2[1] = Elem<DT>::pack(v[2], v[3]);
        *(u32x2*)(dst + 16 * jg) = o2;
      }
    }
    __syncthreads();
    flush_rows(256, [&](int r) -> unsigned char* {
      return p.hq + ((int64_t)(row0 + r) * p.I + nt * 128) * 2;
    });
  } else if (GATED) {
    float h[MT][2][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float amax = 0.0f;
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float gate = acc[mt][jg][i];
          const float up = acc[mt][jg + 2][i];
          const float v = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;  // 1-ulp reciprocal
          h[mt][jg][i] = v;
          amax = fmaxf(amax, fabsf(v));
        }
      }
      amax = fmaxf(amax, __shfl_xor(amax, 16));
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      if (g == 0) red_lds[cg][rbase + 16 * mt + c] = amax;
    }
    __syncthreads();  // row maxima visible; all waves are done with the rings
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int r = rbase + 16 * mt + c;
      const float m = fmaxf(fmaxf(red_lds[0][r], red_lds[1][r]), fmaxf(red_lds[2][r], red_lds[3][r]));
      const float scale = fmaxf(m, kQuantEps) / kFp8Max;
      const float inv = __builtin_amdgcn_rcpf(scale);  // the stored scale stays exact
#pragma unroll
      for (int jg = 0; jg < 2; ++jg) {
        const unsigned int q = pack4_fp8(h[mt][jg][0] * inv, h[mt][jg][1] * inv,
                                         h[mt][jg][2] * inv, h[mt][jg][3] * inv);
        *(unsigned int*)(stage + r * 128 + cg * 32 + 16 * jg + 4 * g) = q;
      }
      if (cg == 0 && g == 0) p.hs[(int64_t)(row0 + r) * (p.I >> 7) + nt] = scale;
    }
    __syncthreads();
    flush_rows(128, [&](int r) -> unsigned char* {
      return p.hq + (int64_t)(row0 + r) * p.I + nt * 128;
    });
  } else {
    __syncthreads();  // all waves are done with the rings (and sid_lds is long visible)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int r = rbase + 16 * mt + c;
      const int sid = sid_lds[r];
      const float rw = sid < p.numel ? p.topk_w[sid] : 0.0f;
      unsigned short* dst = (unsigned short*)stage + r * 256 + cg * 64 + 4 * g;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x2 o2;
        o2[0] = Elem<DT>::pack(acc[mt][j][0] * rw, acc[mt][j][1] * rw);
        o2[1] = Elem<DT>::pack(acc[mt][j][2] * rw, acc[mt][j][3] * rw);
        *(u32x2*)(dst + 16 * j) = o2;
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
  // measured: walking the tiles with resident workgroups pays for the down GEMM (-5 %), not for
  // the gated one (+4 %), which therefore keeps one workgroup per tile
  const uint32_t resident = (uint32_t)persistent_workgroups();
  const uint32_t pgrid = (GATED || grid < resident) ? grid : resident;
#define DLB_LAUNCH_GEMM(DT_) \
  hipLaunchKernelGGL((moe_gemm_fp8_kernel<GATED, DT_, 64, QT>), dim3(pgrid), dim3(256), 0, s, p)
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
  if ((reinterpret_cast<uintptr_t>(hq) & 3u) != 0) return DLB_ERR_UNSUPPORTED;
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
  if ((reinterpret_cast<uintptr_t>(out) & 7u) != 0) return DLB_ERR_UNSUPPORTED;
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
  if ((reinterpret_cast<uintptr_t>(act) & 7u) != 0) return DLB_ERR_UNSUPPORTED;
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
  if ((reinterpret_cast<uintptr_t>(out) & 7u) != 0) return DLB_ERR_UNSUPPORTED;
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
