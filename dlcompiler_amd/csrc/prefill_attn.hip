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
  static constexpr int kRowBytes = D * 2 + 16;      // K: [64][D] + pad
  static constexpr int kBytes = kTileN * kRowBytes;
  static constexpr int vRowBytes = kTileN * 2 + 16;  // V^T: [D][64] + pad
  static constexpr int vBytes = D * vRowBytes;
  static constexpr int stage = kBytes + vBytes;
};

template <int DT, int D>
__global__ __launch_bounds__(kThreads, 2) void prefill_attn_kernel(const PrefillParams p) {
  constexpr int KS = D / 16;  // MFMA k-steps over the head dim for S^T
  constexpr int MT = D / 32;  // 32-row tiles of O^T
  constexpr int KLD = (kTileN * D / 8) / kThreads;  // 16-byte K loads per thread per tile
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
  const int wave_last_row = q0 + 32 * wave + 31;
  const int wave_first_row = q0 + 32 * wave;

  // ---- global -> register staging of one K/V tile
  u32x4 kreg[KLD];
  u32x4 vreg[VLD][4];
  auto load_tile = [&](int t0) {
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int u = i * kThreads + tid;
      const int row = u / DG, cg = u % DG;
      const int key = min(t0 + row, L - 1);
      kreg[i] = *(const u32x4*)(kb + (tok0 + key) * p.k_st + 8 * cg);
    }
#pragma unroll
    for (int i = 0; i < VLD; ++i) {
      const int u = i * kThreads + tid;
      if (VUNITS % kThreads == 0 || u < VUNITS) {
        const int dg = u % DG, kg = u / DG;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = min(t0 + 4 * kg + r, L - 1);
          vreg[i][r] = *(const u32x4*)(vb + (tok0 + key) * p.v_st + 8 * dg);
        }
      }
    }
  };
  auto store_tile = [&](int buf) {
    unsigned char* ks = smem + buf * SM::stage;
    unsigned char* vs = ks + SM::kBytes;
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int u = i * kThreads + tid;
      const int row = u / DG, cg = u % DG;
      *(u32x4*)(ks + row * SM::kRowBytes + cg * 16) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VLD; ++i) {
      const int u = i * kThreads + tid;
      if (VUNITS % kThreads == 0 || u < VUNITS) {
        const int dg = u % DG, kg = u / DG;
        // key = 32*nt + 16*st + 8*a + 4*h + r  ->  position 32*nt + 16*st + 8*h + 4*a + r
        const int unit = ((kg >> 2) << 1) | (kg & 1);  // 4*nt + 2*st + h
        const int half = (kg >> 1) & 1;                // a
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const unsigned int lo01 = __builtin_amdgcn_perm(vreg[i][1][w], vreg[i][0][w], 0x05040100u);
          const unsigned int lo23 = __builtin_amdgcn_perm(vreg[i][3][w], vreg[i][2][w], 0x05040100u);
          const unsigned int hi01 = __builtin_amdgcn_perm(vreg[i][1][w], vreg[i][0][w], 0x07060302u);
          const unsigned int hi23 = __builtin_amdgcn_perm(vreg[i][3][w], vreg[i][2][w], 0x07060302u);
          const int d0 = 8 * dg + 2 * w;
          const int sw = ((d0 >> 4) & 3) << 1;
          unsigned char* row = vs + d0 * SM::vRowBytes + ((unit ^ sw) << 4) + (half << 3);
          *(u32x2*)(row) = u32x2{lo01, lo23};
          *(u32x2*)(row + SM::vRowBytes) = u32x2{hi01, hi23};
        }
      }
    }
  };

  f32x16 o[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[mt][i] = 0.0f;
  float m_run = -__builtin_inff();
  float l_run = 0.0f;  // this lane half's share of the denominator

  load_tile(0);
  store_tile(0);
  __syncthreads();

  for (int j = 0; j < ntiles; ++j) {
    const int t0 = j * kTileN;
    const bool more = (j + 1 < ntiles);
    if (more) load_tile(t0 + kTileN);

    if (t0 <= wave_last_row) {  // wave-uniform: tile not entirely above the diagonal
      const unsigned char* ks = smem + (j & 1) * SM::stage;
      const unsigned char* vs = ks + SM::kBytes;

      // ---- S^T = K . Q^T : two 32-key tiles x 32 queries
      f32x16 s[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[nt][i] = 0.0f;
        const unsigned char* krow = ks + (32 * nt + col) * SM::kRowBytes + 16 * hh;
#pragma unroll
        for (int kstep = 0; kstep < KS; ++kstep) {
          const u32x4 a = *(const u32x4*)(krow + 32 * kstep);
          s[nt] = Mma32<DT>::run(a, qf[kstep], s[nt]);
        }
      }

      // ---- causal mask (diagonal tiles only) and running max, log2 domain
      const bool diag = (t0 + kTileN - 1 > wave_first_row);
      float mloc = -__builtin_inff();
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float x = s[nt][i] * p.scale_log2e;
          if (diag) {
            const int key = t0 + 32 * nt + 8 * (i >> 2) + 4 * hh + (i & 3);
            x = (key <= qrow) ? x : -__builtin_inff();
          }
          s[nt][i] = x;
          mloc = fmaxf(mloc, x);
        }
      }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
      const float m_new = fmaxf(m_run, mloc);  // finite from tile 0 on (key 0 is always visible)
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      float psum = 0.0f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float e = __builtin_amdgcn_exp2f(s[nt][i] - m_new);
          s[nt][i] = e;
          psum += e;
        }
      }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[mt][i] *= alpha;

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
            const int sw = ((d >> 4) & 3) << 1;
            const u32x4 a = *(const u32x4*)(vs + d * SM::vRowBytes + ((unit ^ sw) << 4));
            o[mt] = Mma32<DT>::run(a, pf, o[mt]);
          }
        }
      }
    }

    if (more) store_tile((j + 1) & 1);
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
