// Varlen causal flash-attention prefill for gfx950 (packed [tokens, heads, D] layout, GQA).
//
// Replaces context_attention_fwd + _fwd_kernel
// (python/dlBLAS/dlblas/kernels/prefill_attention.py:39-181): same mathematics -- per
// (sequence, query head, query tile) stream the causal prefix of K/V, QK^T in fp32, online
// softmax, P rounded to the input dtype before P.V -- re-tiled for CDNA4:
//   * a workgroup of 4 wavefronts owns 128 query rows (32 per wave) and walks 64-key K/V tiles
//     that are double-buffered in LDS (global -> registers -> LDS, one barrier per tile);
//   * S^T = K.Q^T and O^T = V^T.P^T on 32x32x16 MFMA.  Working on the transposes puts a query
//     in a lane *column*: the row max/sum are register reductions plus one exchange between
//     the two lane halves, the rescale is a per-lane scalar, and with the key order inside a
//     32-key tile permuted at V-staging time the softmax output registers are already the B
//     operand of the second product (P never crosses lanes);
//   * V is transposed on its way into LDS (4 keys x 8 dims per lane, v_perm + ds_write_b64),
//     K is stored row-major; both are read back as 128-bit MFMA operands;
//   * the exponent runs in base 2 with the softmax scale folded into one FMA;
//   * fully masked tiles are skipped per wave and only diagonal tiles pay for the mask; the
//     heaviest query tiles are launched first.
#include <type_traits>

#include "common.h"

namespace dlb {
namespace {

struct PrefillParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  const int32_t* start_loc;
  const int32_t* seq_len;
  int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;  // token / head strides (elements)
  int Hq, Hkv, group;
  int xcd_heads;  // != 0: remap blockIdx.x so the heads of a KV group share an XCD
  float scale_log2e;
};

template <int DT>
struct Mma32;
template <>
struct Mma32<DLB_DTYPE_BF16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned int pack2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) __bf16 b2;
    f2 f = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, b2));
  }
};
template <>
struct Mma32<DLB_DTYPE_F16> {
  static __device__ __forceinline__ f32x16 run(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned int pack2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    f2 f = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, h2));
  }
};

constexpr int kBlockM = 128;  // query rows per workgroup
constexpr int kTileN = 64;    // keys per LDS tile
constexpr int kThreads = 256;

template <int D>
struct Smem {
  static constexpr int kRowBytes = D * 2;           // K: [64][D], 16-byte chunks XOR-swizzled
  static constexpr int kBytes = kTileN * kRowBytes;
  static constexpr int vRowBytes = kTileN * 2 + 16;  // V^T: [D][64] + pad
  static constexpr int vBytes = D * vRowBytes;
  static constexpr int stage = kBytes + vBytes;
};

#ifndef DLB_PF_OCC
#define DLB_PF_OCC 2
#endif
template <int DT, int D>
__global__ __launch_bounds__(kThreads, DLB_PF_OCC) void prefill_attn_kernel(const PrefillParams p) {
  constexpr int KS = D / 16;  // MFMA k-steps over the head dim for S^T
  constexpr int MT = D / 32;  // 32-row tiles of O^T
  constexpr int VUNITS = (kTileN / 4) * (D / 8);    // (4 keys x 8 dims) units per tile
  constexpr int VLD = (VUNITS + kThreads - 1) / kThreads;
  constexpr int DG = D / 8;
  using SM = Smem<D>;

  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * SM::stage];

  const int seq = blockIdx.z;
  const int L = p.seq_len[seq];
  const int qtile = gridDim.y - 1 - blockIdx.y;  // heaviest tiles first
  const int q0 = qtile * kBlockM;
  if (q0 >= L) return;
  const int64_t tok0 = p.start_loc[seq];
  int head = blockIdx.x;
  if (p.xcd_heads) head = (blockIdx.x & 7) * (p.Hq >> 3) + (blockIdx.x >> 3);
  const int kvh = head / p.group;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int col = lane & 31;  // query column / operand row
  const int hh = lane >> 5;   // lane half

  const unsigned short* qb = (const unsigned short*)p.q;
  const unsigned short* kb = (const unsigned short*)p.k + (int64_t)kvh * p.k_sh;
  const unsigned short* vb = (const unsigned short*)p.v + (int64_t)kvh * p.v_sh;

  // ---- Q^T as B operand: lane (n = query, k = dims 16*ks + 8*hh .. +8), kept in registers
  const int qrow = q0 + 32 * wave + col;
  u32x4 qf[KS];
  {
    const unsigned short* qp =
        qb + (tok0 + min(qrow, L - 1)) * p.q_st + (int64_t)head * p.q_sh + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const u32x4*)(qp + 16 * ks);
  }

  const int kv_end = min(L, q0 + kBlockM);            // keys this workgroup needs
  const int ntiles = (kv_end + kTileN - 1) / kTileN;
  // tiles below this index lie entirely under the diagonal for every wave of the workgroup
  // (q0 is a multiple of 128): no mask, no clamping of key rows
  const int nfull = q0 / kTileN;
  const int wave_last_row = q0 + 32 * wave + 31;

  // ---- global -> register staging of one K/V tile.  Per-thread base pointers are formed
  // once; a tile adds a workgroup-uniform offset.  CLAMP (tiles that may run past the
  // sequence) redirects rows >= L to row L-1 so nothing outside the sequence is read.
  // K goes global -> LDS directly (global_load_lds_dwordx4: lane l's 16 bytes land at
  // base + 16*l, so one wave instruction fills 1 KB = 1024 / (2*D) rows).  Rows are stored
  // unpadded; bank conflicts are avoided by letting lane (row r, position c) fetch global
  // chunk c ^ (r & 15): a reader that wants chunk c of row r reads position c ^ (r & 15).
  constexpr int KRPI = 1024 / (2 * D);            // rows per wave instruction
  constexpr int KINS = kTileN / KRPI / 4;         // instructions per wave and tile
  const int k_lrow = lane / DG;                   // row inside an instruction
  const int k_pos = lane % DG;                    // 16-byte position inside the row
  const unsigned char* kbytes = (const unsigned char*)kb;
  const unsigned char* vbase = (const unsigned char*)vb + ((tok0 + 4 * (tid / DG)) * p.v_st + 8 * (tid % DG)) * 2;
  const int64_t k_row_bytes = p.k_st * 2, v_row_bytes = p.v_st * 2;
  const bool v_active = (VUNITS >= kThreads) || (tid < VUNITS);
  u32x4 vreg[4];
  static_assert(VLD == 1, "one (4 keys x 8 dims) V unit per thread");
  auto load_tile = [&](auto clamp_tag, int t0, int buf) {
    constexpr bool CLAMP = decltype(clamp_tag)::value;
    unsigned char* ks = smem + buf * SM::stage;
#pragma unroll
    for (int i = 0; i < KINS; ++i) {
      const int q = 4 * i + wave;                 // which 1 KB slice of the tile
      const int r = q * KRPI + k_lrow;            // key row inside the tile
      int key = t0 + r;
      if (CLAMP) key = min(key, L - 1);
      const unsigned char* src = kbytes + (tok0 + key) * k_row_bytes + ((k_pos ^ (r & (DG - 1))) << 4);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                       (__attribute__((address_space(3))) void*)(ks + q * 1024),
                                       16, 0, 0);
    }
    if (v_active) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int row = t0 + r;  // + 4 * (tid / DG) is in vbase
        if (CLAMP) row = min(row + 4 * (tid / DG), L - 1) - 4 * (tid / DG);
        vreg[r] = *(const u32x4*)(vbase + row * v_row_bytes);
      }
    }
  };
  // LDS addresses of this thread's staging slots (tile-independent)
  const int st_kg = tid / DG, st_dg = tid % DG;
  // key = 32*nt + 16*st + 8*a + 4*h + r  ->  position 32*nt + 16*st + 8*h + 4*a + r
  const int st_unit = ((st_kg >> 2) << 1) | (st_kg & 1);  // 16-byte unit 4*nt + 2*st + h
  const int st_half = (st_kg >> 1) & 1;                   // 8-byte half a
  auto store_tile = [&](int buf) {
    unsigned char* vs = smem + buf * SM::stage + SM::kBytes;
    if (v_active) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned int lo01 = __builtin_amdgcn_perm(vreg[1][w], vreg[0][w], 0x05040100u);
        const unsigned int lo23 = __builtin_amdgcn_perm(vreg[3][w], vreg[2][w], 0x05040100u);
        const unsigned int hi01 = __builtin_amdgcn_perm(vreg[1][w], vreg[0][w], 0x07060302u);
        const unsigned int hi23 = __builtin_amdgcn_perm(vreg[3][w], vreg[2][w], 0x07060302u);
        const int d0 = 8 * st_dg + 2 * w;
        const int sw = (d0 >> 4) & 7;  // same for d0 and d0 + 1; spreads the 16 dim groups
        unsigned char* row = vs + d0 * SM::vRowBytes + ((st_unit ^ sw) << 4) + (st_half << 3);
        *(u32x2*)(row) = u32x2{lo01, lo23};
        *(u32x2*)(row + SM::vRowBytes) = u32x2{hi01, hi23};
      }
    }
  };

  f32x16 o[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[mt][i] = 0.0f;
  // m_run is the exponent reference in the log2 domain.  It follows the running maximum
  // lazily: the accumulators are rescaled only when a row maximum exceeds it by more than
  // kRescaleGap, so between rescales probabilities stay below 2^kRescaleGap -- exact in the
  // end (the same factor cancels in O / l), and it removes the per-tile rescale of O.
  constexpr float kRescaleGap = 8.0f;
  float m_run = -__builtin_inff();
  float l_run = 0.0f;  // this lane half's share of the denominator
  const float cs = p.scale_log2e;

  // one K/V tile against this wave's 32 queries; MASK: apply the causal mask
  auto process_tile = [&](auto mask_tag, int j) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const int t0 = j * kTileN;
    if (MASK && t0 > wave_last_row) return;  // wave-uniform: tile entirely above the diagonal
    const unsigned char* ks = smem + (j & 1) * SM::stage;
    const unsigned char* vs = ks + SM::kBytes;

    // ---- S^T = K . Q^T : two 32-key tiles x 32 queries (raw scores)
    f32x16 s[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[nt][i] = 0.0f;
      const int krow_i = 32 * nt + col;
      const unsigned char* krow = ks + krow_i * SM::kRowBytes;
      const int ksw = krow_i & (DG - 1);
#pragma unroll
      for (int kstep = 0; kstep < KS; ++kstep) {
        const u32x4 a = *(const u32x4*)(krow + (((2 * kstep + hh) ^ ksw) << 4));
        s[nt] = Mma32<DT>::run(a, qf[kstep], s[nt]);
      }
    }

    // ---- causal mask and tile maximum of the raw scores (scale > 0 commutes with max)
    float mloc = -__builtin_inff();
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (MASK) {
          const int key = t0 + 32 * nt + 8 * (i >> 2) + 4 * hh + (i & 3);
          s[nt][i] = (key <= qrow) ? s[nt][i] : -__builtin_inff();
        }
        mloc = fmaxf(mloc, s[nt][i]);
      }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32)) * cs;
    if (__any(mloc > m_run + kRescaleGap)) {
      const float m_new = fmaxf(m_run, mloc);  // finite from tile 0 on (key 0 is visible)
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[mt][i] *= alpha;
    }
    float psum = 0.0f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nt][i], cs, -m_run));
        s[nt][i] = e;
        psum += e;
      }
    }
    l_run += psum;

    // ---- O^T += V^T . P^T ; step (nt, st) consumes registers 8*st .. 8*st+7 of s[nt]
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        u32x4 pf;
        pf[0] = Mma32<DT>::pack2(s[nt][8 * st + 0], s[nt][8 * st + 1]);
        pf[1] = Mma32<DT>::pack2(s[nt][8 * st + 2], s[nt][8 * st + 3]);
        pf[2] = Mma32<DT>::pack2(s[nt][8 * st + 4], s[nt][8 * st + 5]);
        pf[3] = Mma32<DT>::pack2(s[nt][8 * st + 6], s[nt][8 * st + 7]);
        const int unit = 4 * nt + 2 * st + hh;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int d = 32 * mt + col;
          const int sw = (d >> 4) & 7;
          const u32x4 a = *(const u32x4*)(vs + d * SM::vRowBytes + ((unit ^ sw) << 4));
          o[mt] = Mma32<DT>::run(a, pf, o[mt]);
        }
      }
    }
  };

  using NoClamp = std::integral_constant<bool, false>;
  using Clamp = std::integral_constant<bool, true>;
  // vmcnt(0): the direct-to-LDS loads of this wave have landed before the barrier publishes
  // the buffer (encoding: vmcnt = 0, expcnt / lgkmcnt left at their maxima)
  auto wait_dma = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };
  if (nfull > 0) load_tile(NoClamp{}, 0, 0); else load_tile(Clamp{}, 0, 0);
  store_tile(0);
  wait_dma();
  __syncthreads();

  int j = 0;
  // tiles under the diagonal whose successor is also under it: nothing to mask or clamp
  for (; j + 1 < nfull; ++j) {
    load_tile(NoClamp{}, (j + 1) * kTileN, (j + 1) & 1);
    process_tile(std::integral_constant<bool, false>{}, j);
    store_tile((j + 1) & 1);
    wait_dma();
    __syncthreads();
  }
  // last unmasked tile (its successor may run past the sequence), then the diagonal tiles
  for (; j < ntiles; ++j) {
    const bool more = (j + 1 < ntiles);
    if (more) load_tile(Clamp{}, (j + 1) * kTileN, (j + 1) & 1);
    if (j < nfull) process_tile(std::integral_constant<bool, false>{}, j);
    else process_tile(std::integral_constant<bool, true>{}, j);
    if (more) store_tile((j + 1) & 1);
    wait_dma();
    __syncthreads();
  }

  // ---- epilogue: normalise and store O (lane holds 4 consecutive dims per register quad)
  l_run += __shfl_xor(l_run, 32);
  if (qrow < L) {
    const float inv = 1.0f / l_run;
    unsigned short* op = (unsigned short*)p.o + (tok0 + qrow) * p.o_st + (int64_t)head * p.o_sh;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 w;
        w[0] = Mma32<DT>::pack2(o[mt][4 * qd + 0] * inv, o[mt][4 * qd + 1] * inv);
        w[1] = Mma32<DT>::pack2(o[mt][4 * qd + 2] * inv, o[mt][4 * qd + 3] * inv);
        *(u32x2*)(op + 32 * mt + 8 * qd + 4 * hh) = w;
      }
    }
  }
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_prefill_attn_varlen(const void* q, const void* k, const void* v, void* o,
                                       const int32_t* start_loc, const int32_t* seq_len, int B,
                                       int Hq, int Hkv, int D, int max_len, int64_t q_stride_tok,
                                       int64_t q_stride_head, int64_t k_stride_tok,
                                       int64_t k_stride_head, int64_t v_stride_tok,
                                       int64_t v_stride_head, int64_t o_stride_tok,
                                       int64_t o_stride_head, float sm_scale, int dtype,
                                       void* stream) {
  using namespace dlb;
  if (B < 0 || Hq < 1 || Hkv < 1 || D < 1 || max_len < 0) return DLB_ERR_BAD_ARG;
  if (Hq % Hkv != 0) return DLB_ERR_BAD_ARG;
  if (B == 0 || max_len == 0) return DLB_OK;
  if (!q || !k || !v || !o || !start_loc || !seq_len) return DLB_ERR_BAD_ARG;
  if (D != 64 && D != 128) return DLB_ERR_UNSUPPORTED;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) ||
      (reinterpret_cast<uintptr_t>(o) & 7u) != 0)
    return DLB_ERR_UNSUPPORTED;
  const int64_t in_strides[] = {q_stride_tok, q_stride_head, k_stride_tok,
                                k_stride_head, v_stride_tok, v_stride_head};
  for (int64_t sd : in_strides)
    if (sd % 8 != 0) return DLB_ERR_UNSUPPORTED;
  if (o_stride_tok % 4 != 0 || o_stride_head % 4 != 0) return DLB_ERR_UNSUPPORTED;
  if (B > 65535) return DLB_ERR_UNSUPPORTED;

  PrefillParams p;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = o;
  p.start_loc = start_loc;
  p.seq_len = seq_len;
  p.q_st = q_stride_tok;
  p.q_sh = q_stride_head;
  p.k_st = k_stride_tok;
  p.k_sh = k_stride_head;
  p.v_st = v_stride_tok;
  p.v_sh = v_stride_head;
  p.o_st = o_stride_tok;
  p.o_sh = o_stride_head;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.group = Hq / Hkv;
  // workgroups are dealt round-robin to the 8 XCDs by linear id; with Hq % 8 == 0 the
  // remap in the kernel puts heads {x, x+8, ...} -> consecutive heads on one XCD so a KV
  // group's four query heads hit the same L2.
  p.xcd_heads = (Hq % 8 == 0 && Hq >= 16) ? 1 : 0;
  p.scale_log2e = sm_scale * 1.4426950408889634f;

  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)Hq, (uint32_t)ceil_div(max_len, kBlockM), (uint32_t)B);
  if (grid.y > 65535) return DLB_ERR_UNSUPPORTED;
#define DLB_LAUNCH_PREFILL(DT_, D_) \
  hipLaunchKernelGGL((prefill_attn_kernel<DT_, D_>), grid, dim3(kThreads), 0, s, p)
  if (dtype == DLB_DTYPE_BF16) {
    if (D == 128) DLB_LAUNCH_PREFILL(DLB_DTYPE_BF16, 128);
    else DLB_LAUNCH_PREFILL(DLB_DTYPE_BF16, 64);
  } else {
    if (D == 128) DLB_LAUNCH_PREFILL(DLB_DTYPE_F16, 128);
    else DLB_LAUNCH_PREFILL(DLB_DTYPE_F16, 64);
  }
#undef DLB_LAUNCH_PREFILL
  return launch_status();
}
