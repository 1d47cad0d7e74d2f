// Varlen causal flash-attention prefill for gfx950 (packed [tokens, heads, D] layout, GQA).
//
// Replaces context_attention_fwd + _fwd_kernel
// (python/dlBLAS/dlblas/kernels/prefill_attention.py:39-181): same mathematics -- per
// (sequence, query head, query tile) stream the causal prefix of K/V, QK^T in fp32, online
// softmax, P rounded to the input dtype before P.V -- re-tiled for CDNA4:
//   * a workgroup of 4 wavefronts owns 128 query rows (32 per wave) and walks 64-key K/V tiles
//     that are double-buffered in LDS (copied global -> LDS directly, one barrier per tile);
//   * S^T = K.Q^T and O^T = V^T.P^T on 32x32x16 MFMA.  Working on the transposes puts a query
//     in a lane *column*: the row max/sum are register reductions plus one exchange between
//     the two lane halves, the rescale is a per-lane scalar, and the softmax output registers
//     are already the B operand of the second product (P never crosses lanes): the V^T
//     operand is simply fetched in the key order those registers have;
//   * K and V both sit row-major in LDS.  K fragments are 128-bit reads; V^T fragments come
//     from ds_read_b64_tr_b16, which hands lane l of a 16-lane group column l of a 4-row x
//     16-column block (rows supplied by lanes 4j .. 4j+3), i.e. the transpose happens in the
//     LDS read and V never passes through registers on its way in;
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
  IdxArray start_loc;
  IdxArray seq_len;
  int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, o_st, o_sh;  // token / head strides (elements)
  int Hq, Hkv, group;
  int xcd_heads;  // != 0: remap blockIdx.x so the heads of a KV group share an XCD
  float scale_log2e;
  // paged K/V (PAGED kernels): k/v point at caches [pages, page, Hkv, D]; *_st is the slot
  // stride, *_sp the page stride; sequence s reads pages block_table[s][.] and its queries sit
  // at context positions kv_len[s] - seq_len[s] + i
  IdxArray kv_len;
  IdxArray block_table;
  int64_t bt_stride, k_sp, v_sp;
  int page, page_shift;
  int dk, dv;  // real key / value head sizes (<= the padded size D the kernel is built for)
  // generic masking (both layouts): sliding window (> 0) and logit soft-cap (> 0)
  int window;
  float softcap, sm_scale;
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
  static constexpr int vBytes = kBytes;              // V: [64][D], 16-byte chunks XOR-swizzled
  static constexpr int stage = kBytes + vBytes;
};

// D is the padded head size the kernel is built for (64 or 128).  RAGGED: the real key size dk
// and / or value size dv is smaller (any multiple of 8): the query dims past dk are loaded as
// zeros, so the key bytes staged for those dims do not count -- their copies are redirected to
// the row's first 16 bytes to stay inside the tensor -- and value dims past dv (redirected
// likewise) only produce output dims that are never stored.  The reference handles odd head
// sizes by splitting them into power-of-two blocks with masked loads
// (python/dlBLAS/dlblas/kernels/paged_attention.py:531-539).
// PAGED: 0 = packed K/V; 1 = paged, every K/V row looks up its own page (any page size); 2 = paged
// with pages that are whole multiples of the 64-key tile: a tile lies in one page, so its page
// number is one wave-uniform look-up and the copies are addressed as in the packed layout (a
// scalar base per tile plus constant lane offsets).
template <int DT, int D, int PAGED, bool RAGGED>
__global__ __launch_bounds__(kThreads, D > 128 ? 1 : 2) void prefill_attn_kernel(const PrefillParams p) {
  constexpr int KS = D / 16;  // MFMA k-steps over the head dim for S^T
  constexpr int MT = D / 32;  // 32-row tiles of O^T
  constexpr int DG = D / 8;
  using SM = Smem<D>;

  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * SM::stage];

  // The grid runs over (head, query tile, sequence), tile index reversed: what an XCD holds at
  // any time is the query tiles of ONE sequence's heads of ONE KV group (see the head remap
  // below), i.e. workgroups that stream the same K/V rows, which its L2 then serves after the
  // first read; within a sequence the heaviest (last) tiles start first.
  // Paged (chunked) prefill: a sequence's cost is set by its history, which differs widely
  // between the sequences of a batch while the grid holds only a few workgroups per slot, so
  // the sequences are walked longest context first (blockIdx.z = rank, not index): the long
  // ones start in the first round and the short ones fill in behind them.  (The packed layout
  // has many workgroups per slot and gains nothing from the ranking: measured 1.5 % slower.)
  int seq = blockIdx.z;
  if (PAGED && gridDim.z > 1 && gridDim.z <= kThreads) {
    __shared__ int32_t rank_key[kThreads];
    __shared__ int32_t rank_seq;
    const int nb = gridDim.z;
    const int t = threadIdx.x;
    const int key = t < nb ? p.kv_len[t] : 0;
    rank_key[t] = key;
    __syncthreads();
    if (t < nb) {
      int rank = 0;
      for (int j = 0; j < nb; ++j) {
        const int kj = rank_key[j];
        rank += (kj > key || (kj == key && j < t)) ? 1 : 0;
      }
      if (rank == (int)blockIdx.z) rank_seq = t;  // ranks are a permutation: exactly one writer
    }
    __syncthreads();
    seq = __builtin_amdgcn_readfirstlane(rank_seq);
  }
  const int L = p.seq_len[seq];
  const int qtile = gridDim.y - 1 - blockIdx.y;  // heaviest first
  const int q0 = qtile * kBlockM;
  if (q0 >= L) return;
  const int64_t tok0 = p.start_loc[seq];
  // context seen by this sequence: kv_total keys, the queries are its last L positions
  const int kv_total = PAGED ? p.kv_len[seq] : L;
  const int hist = kv_total - L;
  if (PAGED && hist < 0) return;  // inconsistent lengths: nothing sensible to compute
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
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = u32x4{0u, 0u, 0u, 0u};
      if (!RAGGED || 16 * ks + 8 * hh < p.dk) qf[ks] = *(const u32x4*)(qp + 16 * ks);
    }
  }

  const int kv_end = min(kv_total, hist + q0 + kBlockM);  // keys this workgroup needs
  const int ntiles = (kv_end + kTileN - 1) / kTileN;
  // window / soft-cap requests take the masked path for every tile
  // (only the paged entry point exposes them; the packed kernel compiles them out)
  const int window = PAGED ? p.window : -1;
  const float softcap = PAGED ? p.softcap : -1.0f;
  const bool generic = (window > 0) || (softcap > 0.0f);
  // tiles below this index lie entirely under the diagonal for every wave of the workgroup
  // (all 64 keys <= position of row q0): no mask, no clamping of key rows
  const int nfull = generic ? 0 : (hist + q0 + 1) / kTileN;
  // first tile that can hold a visible key (sliding window)
  const int jfirst = window > 0 ? max(hist + q0 - window, 0) / kTileN : 0;
  const int qpos = hist + qrow;                          // context position of this lane's query
  const int wave_last_pos = hist + q0 + 32 * wave + 31;

  // ---- global -> LDS staging of one K/V tile.  Per-thread base pointers are formed once; a
  // tile adds a workgroup-uniform offset.  CLAMP (tiles that may run past the sequence)
  // redirects rows >= kv_total to the last row so nothing outside the sequence is read.
  // Both operands go global -> LDS directly (global_load_lds_dwordx4: lane l's 16 bytes land
  // at base + 16*l, so one wave instruction fills 1 KB = 1024 / (2*D) rows).  Rows are stored
  // unpadded; bank conflicts are avoided by permuting which 16-byte chunk of its row a lane
  // fetches: position c of row r holds chunk c ^ swz(r), so a reader that wants chunk c of
  // row r reads position c ^ swz(r).  K: swz(r) = r mod DG (128-bit fragment reads, one row
  // per lane).  V: swz(r) spreads the 4 (or 8) rows that one transposing read touches over
  // all banks.
  constexpr int KRPI = 1024 / (2 * D);            // rows per wave instruction
  constexpr int KINS = kTileN / KRPI / 4;         // instructions per wave, tile and operand
  const int k_lrow = lane / DG;                   // row inside an instruction
  const int k_pos = lane % DG;                    // 16-byte position inside the row
  const unsigned char* kbytes = (const unsigned char*)kb;
  const unsigned char* vbytes = (const unsigned char*)vb;
  const int64_t k_row_bytes = p.k_st * 2, v_row_bytes = p.v_st * 2;
  const IdxArray bt = {PAGED ? p.block_table.p + (((int64_t)seq * p.bt_stride) << p.block_table.sh) : nullptr,
                       p.block_table.sh};
  // V chunk swizzle of row r (depends on r mod 8 only)
  auto v_swz = [](int r) -> int {
    return D == 128 ? (((r & 3) << 2) | (((r >> 2) & 1) << 1))
                    : ((((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1));
  };
  // byte offset inside its source row of the 16-byte chunk this lane copies into position k_pos
  // of row r (the swizzle undone; chunks past the real head size fetch the row's first chunk)
  auto k_chunk = [&](int r) -> unsigned int {
    const int c = k_pos ^ (r & (DG - 1));
    return (unsigned int)((RAGGED && 8 * c >= p.dk) ? 0 : c) << 4;
  };
  auto v_chunk = [&](int r) -> unsigned int {
    const int c = k_pos ^ v_swz(r);
    return (unsigned int)((RAGGED && 8 * c >= p.dv) ? 0 : c) << 4;
  };
  // paged layout: the page ids of the rows this lane copies are fetched one tile ahead of the
  // copy that needs them, so the block-table latency never sits in front of a tile's copies
  int pg_next[KINS];
  int pg_tile = 0;  // PAGED == 2: the page of the next tile to stage (wave-uniform)
  auto fetch_pages = [&](int t0) {
    if (PAGED == 2) {
      const int key = min(t0, kv_total - 1);
      pg_tile = bt[p.page_shift >= 0 ? (key >> p.page_shift) : (key / p.page)];
      return;
    }
#pragma unroll
    for (int i = 0; i < KINS; ++i) {
      const int key = min(t0 + (4 * i + wave) * KRPI + k_lrow, kv_total - 1);
      pg_next[i] = bt[p.page_shift >= 0 ? (key >> p.page_shift) : (key / p.page)];
    }
  };
  const unsigned int smem_base = lds_addr(smem) + wave * 1024;  // + q * 1024 with q = 4*i + wave
  // source addresses and LDS targets of the copies of the tile being staged: prepare_tile
  // computes them, issue_copy(n) sends copy n of 2 * KINS (K and V slices alternate)
  // Packed layout: a copy's address is a tile base in scalar registers plus a 32-bit lane
  // offset that does not change from tile to tile (row inside the tile x row pitch + chunk),
  // so an unclamped tile costs no vector arithmetic.  Paged layout: every row has its own
  // page, so full 64-bit lane addresses are formed.
  const unsigned char* ksrc[KINS];
  const unsigned char* vsrc[KINS];
  unsigned int koff[KINS], voff[KINS], koff0[KINS], voff0[KINS];
  const unsigned char* kbase = nullptr;
  const unsigned char* vbase = nullptr;
#pragma unroll
  for (int i = 0; i < KINS; ++i) {
    const int r = (4 * i + wave) * KRPI + k_lrow;
    koff0[i] = (unsigned int)(r * k_row_bytes) + k_chunk(r);
    voff0[i] = (unsigned int)(r * v_row_bytes) + v_chunk(r);
  }
  unsigned int stage_dst = 0;
  auto prepare_tile = [&](auto clamp_tag, int t0, int buf) {
    constexpr bool CLAMP = decltype(clamp_tag)::value;
    stage_dst = smem_base + buf * SM::stage;
    if (!PAGED) {
      kbase = uniform_ptr(kbytes + (tok0 + t0) * k_row_bytes);
      vbase = uniform_ptr(vbytes + (tok0 + t0) * v_row_bytes);
    }
    if (PAGED == 2) {
      // t0 is a multiple of the tile and the page a multiple of the tile: slot of the tile's
      // first key inside its page (a tile whose first key lies past the context is never staged)
      const int pi = p.page_shift >= 0 ? (t0 >> p.page_shift) : (t0 / p.page);
      const int64_t pg = __builtin_amdgcn_readfirstlane(pg_tile);
      const int64_t slot0 = t0 - pi * p.page;
      kbase = uniform_ptr(kbytes + (pg * p.k_sp + slot0 * p.k_st) * 2);
      vbase = uniform_ptr(vbytes + (pg * p.v_sp + slot0 * p.v_st) * 2);
    }
#pragma unroll
    for (int i = 0; i < KINS; ++i) {
      const int r = (4 * i + wave) * KRPI + k_lrow;  // key row inside the tile
      if (PAGED == 1) {
        int key = t0 + r;
        if (CLAMP) key = min(key, kv_total - 1);
        const int pi = p.page_shift >= 0 ? (key >> p.page_shift) : (key / p.page);
        const int64_t slot = key - pi * p.page;
        ksrc[i] = kbytes + ((int64_t)pg_next[i] * p.k_sp + slot * p.k_st) * 2 + k_chunk(r);
        vsrc[i] = vbytes + ((int64_t)pg_next[i] * p.v_sp + slot * p.v_st) * 2 + v_chunk(r);
      } else if (CLAMP) {
        const int rc = min(r, kv_total - 1 - t0);  // >= 0: a staged tile starts inside the context
        koff[i] = (unsigned int)(rc * k_row_bytes) + k_chunk(r);
        voff[i] = (unsigned int)(rc * v_row_bytes) + v_chunk(r);
      } else {
        koff[i] = koff0[i];
        voff[i] = voff0[i];
      }
    }
    if (PAGED) fetch_pages(t0 + kTileN);  // consumed by the next prepare_tile
  };
  auto issue_copy = [&](int n) {
    const int i = n >> 1;  // 1 KB slice 4*i + wave of the tile
    const unsigned int dst = stage_dst + (n & 1) * SM::kBytes + i * 4096;
    if (PAGED == 1) dma16_global_to_lds((n & 1) ? vsrc[i] : ksrc[i], dst);
    else if (n & 1) dma16_global_to_lds(vbase, voff[i], dst);
    else dma16_global_to_lds(kbase, koff[i], dst);
  };
  auto load_tile = [&](auto clamp_tag, int t0, int buf) {
    prepare_tile(clamp_tag, t0, buf);
#pragma unroll
    for (int n = 0; n < 2 * KINS; ++n) issue_copy(n);
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

  // byte offsets of this lane's transposing V reads inside a tile, one per 32-dim block
  int v_off[MT];
  {
    const int s16 = lane & 15, dhalf = (lane >> 4) & 1;
    const int r = 4 * hh + (s16 >> 2);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      v_off[mt] = r * SM::kRowBytes +
                  (((4 * mt + 2 * dhalf + ((s16 >> 1) & 1)) ^ v_swz(r)) << 4) + 8 * (s16 & 1);
  }

  // one K/V tile against this wave's 32 queries; MASK: apply the causal mask
  // COPY: the copies of the tile prepared by prepare_tile go out between the S^T MFMAs, one per
  // k-step, instead of as one burst that would hold up this wave's instruction stream
  auto process_tile = [&](auto mask_tag, auto copy_tag, int j) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr bool COPY = decltype(copy_tag)::value;
    static_assert(2 * KINS == KS, "one copy per k-step");
    const int t0 = j * kTileN;
    if (MASK && t0 > wave_last_pos) return;  // wave-uniform: tile entirely above the diagonal
    if (MASK && window > 0 && t0 + kTileN - 1 < wave_last_pos - 31 - window) return;  // below the window
    const unsigned char* ks = smem + (j & 1) * SM::stage;
    const unsigned char* vs = ks + SM::kBytes;

    // ---- S^T = K . Q^T : two 32-key tiles x 32 queries (raw scores)
    // k-step outer, key tile inner: two independent accumulator chains, and the K fragments
    // are fetched from LDS two k-steps ahead of the MFMAs that consume them
    f32x16 s[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[nt][i] = 0.0f;
    // MFMA-dense phase: let this wave's issue win over the other wave of the SIMD, whose
    // softmax arithmetic then fills the gaps while the matrix pipe is busy
    __builtin_amdgcn_s_setprio(1);
    {
      const unsigned char* krow0 = ks + col * SM::kRowBytes;
      const unsigned char* krow1 = ks + (32 + col) * SM::kRowBytes;
      const int ksw = col & (DG - 1);  // (32 + col) & (DG - 1) is the same
      auto ldk = [&](int kstep, u32x4 (&a)[2]) {
        const int off = ((2 * kstep + hh) ^ ksw) << 4;
        a[0] = *(const u32x4*)(krow0 + off);
        a[1] = *(const u32x4*)(krow1 + off);
      };
      constexpr int kAhead = 2;
      u32x4 ka[kAhead + 1][2];
#pragma unroll
      for (int q = 0; q < kAhead; ++q) ldk(q, ka[q]);
#pragma unroll
      for (int kstep = 0; kstep < KS; ++kstep) {
        if (kstep + kAhead < KS) ldk(kstep + kAhead, ka[(kstep + kAhead) % (kAhead + 1)]);
        if (COPY) issue_copy(kstep);
        __builtin_amdgcn_sched_barrier(0);  // keep the fetch ahead of the MFMAs (it would be sunk)
        s[0] = Mma32<DT>::run(ka[kstep % (kAhead + 1)][0], qf[kstep], s[0]);
        s[1] = Mma32<DT>::run(ka[kstep % (kAhead + 1)][1], qf[kstep], s[1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    __builtin_amdgcn_s_setprio(0);
    // ---- causal mask and tile maximum of the raw scores (scale > 0 commutes with max)
    float mpart[2] = {-__builtin_inff(), -__builtin_inff()};  // two independent chains
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (MASK) {
          const int key = t0 + 32 * nt + 8 * (i >> 2) + 4 * hh + (i & 3);
          float x = s[nt][i];
          if (softcap > 0.0f)  // cap * tanh(x * scale / cap), kept in raw-score units
            x = tanhf(x * (p.sm_scale / softcap)) * (softcap / p.sm_scale);
          bool vis = key <= qpos;
          if (window > 0) vis = vis && (key >= qpos - window);
          s[nt][i] = vis ? x : -__builtin_inff();
        }
        mpart[nt] = fmaxf(mpart[nt], s[nt][i]);
      }
    }
    // (the scale is applied here, to fp32 scores, as the reference does: folded into Q -- which
    // would save the multiply-add below -- it is rounded to the element type, an error that
    // grows with the score and reaches several percent of the probabilities at |score| ~ 100)
    const float mloc = max_xor32(fmaxf(mpart[0], mpart[1])) * cs;
    if (__any(mloc > m_run + kRescaleGap)) {
      const float m_new = fmaxf(m_run, mloc);  // finite from tile 0 on (key 0 is visible)
      // (a fully masked row under a sliding window keeps m_new = -inf: leave it untouched)
      const float alpha = (MASK && PAGED && m_new == -__builtin_inff()) ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[mt][i] *= alpha;
    }
    // a row whose keys so far were all masked (sliding window) still has m_run = -inf
    const float m_ref = (MASK && PAGED && m_run == -__builtin_inff()) ? 0.0f : m_run;
    float psum = 0.0f;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nt][i], cs, -m_ref));
        s[nt][i] = e;
        psum += e;
      }
    }
    l_run += psum;

    // ---- O^T += V^T . P^T ; step (nt, st) consumes registers 8*st .. 8*st+7 of s[nt], which
    // belong to keys 32*nt + 16*st + 8*a + 4*hh + r (slot e = 4*a + r).  The A operand wants,
    // for dim d = 32*mt + col, the same 8 keys: two transposing reads (a = 0, 1), in each of
    // which lane s of 16-lane group g supplies row 4*hh + (s >> 2) (+ the step's key base),
    // dims 32*mt + 16*(g & 1) + 4*(s & 3) .. +3.
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        u32x4 pf;
        pf[0] = Mma32<DT>::pack2(s[nt][8 * st + 0], s[nt][8 * st + 1]);
        pf[1] = Mma32<DT>::pack2(s[nt][8 * st + 2], s[nt][8 * st + 3]);
        pf[2] = Mma32<DT>::pack2(s[nt][8 * st + 4], s[nt][8 * st + 5]);
        pf[3] = Mma32<DT>::pack2(s[nt][8 * st + 6], s[nt][8 * st + 7]);
        const unsigned char* vstep = vs + (32 * nt + 16 * st) * SM::kRowBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const u32x2 lo = lds_read_tr16(vstep + v_off[mt]);
          const u32x2 hi = lds_read_tr16(vstep + v_off[mt] + 8 * SM::kRowBytes);
          o[mt] = Mma32<DT>::run(u32x4{lo[0], lo[1], hi[0], hi[1]}, pf, o[mt]);
        }
      }
    }
  };

  using NoClamp = std::integral_constant<bool, false>;
  using Clamp = std::integral_constant<bool, true>;
  // vmcnt(0): the direct-to-LDS loads of this wave have landed before the barrier publishes
  // the buffer (encoding: vmcnt = 0, expcnt / lgkmcnt left at their maxima)
  auto wait_dma = [&]() { __builtin_amdgcn_s_waitcnt(0x0F70); };
  int j = jfirst;
  if (PAGED) fetch_pages(j * kTileN);
  if (j < nfull) load_tile(NoClamp{}, j * kTileN, j & 1); else load_tile(Clamp{}, j * kTileN, j & 1);
  wait_dma();
  __syncthreads();

  // tiles under the diagonal whose successor is also under it: nothing to mask or clamp
  using Yes = std::integral_constant<bool, true>;
  using No = std::integral_constant<bool, false>;
  for (; j + 1 < nfull; ++j) {
    prepare_tile(NoClamp{}, (j + 1) * kTileN, (j + 1) & 1);
    process_tile(No{}, Yes{}, j);
    wait_dma();
    __syncthreads();
  }
  // last unmasked tile (its successor may run past the sequence), then the diagonal tiles
  for (; j < ntiles; ++j) {
    const bool more = (j + 1 < ntiles);
    if (more) load_tile(Clamp{}, (j + 1) * kTileN, (j + 1) & 1);
    // a diagonal tile still lies entirely under the diagonal for the waves further down
    const bool wave_full = !generic && (j + 1) * kTileN - 1 <= hist + q0 + 32 * wave;
    if (j < nfull || wave_full) process_tile(No{}, No{}, j);
    else process_tile(Yes{}, No{}, j);
    wait_dma();
    __syncthreads();
  }

  // ---- epilogue: normalise and store O (lane holds 4 consecutive dims per register quad)
  l_run += __shfl_xor(l_run, 32);
  if (qrow < L) {
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    unsigned short* op = (unsigned short*)p.o + (tok0 + qrow) * p.o_st + (int64_t)head * p.o_sh;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 w;
        w[0] = Mma32<DT>::pack2(o[mt][4 * qd + 0] * inv, o[mt][4 * qd + 1] * inv);
        w[1] = Mma32<DT>::pack2(o[mt][4 * qd + 2] * inv, o[mt][4 * qd + 3] * inv);
        if (!RAGGED || 32 * mt + 8 * qd + 4 * hh < p.dv) *(u32x2*)(op + 32 * mt + 8 * qd + 4 * hh) = w;
      }
    }
  }
}

}  // namespace
}  // namespace dlb

namespace dlb {
namespace {

// Shared argument checks and launch of both entry points; the paged fields of `p` are already
// filled in (or zeroed) by the caller.
int launch_prefill(PrefillParams& p, bool paged, int B, int Hq, int Hkv, int Dk, int Dv, int max_len,
                   float sm_scale, int dtype, void* stream) {
  if (Dk % 8 != 0 || Dv % 8 != 0 || Dk > 256 || Dv > 256) return DLB_ERR_UNSUPPORTED;
  // head size the kernel instance is built for; past 128 there is one instance, for 256, that
  // takes every size on its ragged path (one workgroup per CU, one wave per SIMD: the 128 output
  // accumulators and the 64 query registers of a lane leave no room for a second wave)
  const int D = (Dk <= 64 && Dv <= 64) ? 64 : (Dk <= 128 && Dv <= 128) ? 128 : 256;
  const bool ragged = Dk != D || Dv != D || D == 256;
  p.dk = Dk;
  p.dv = Dv;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
  if (!aligned16(p.q) || !aligned16(p.k) || !aligned16(p.v) ||
      (reinterpret_cast<uintptr_t>(p.o) & 7u) != 0)
    return DLB_ERR_UNSUPPORTED;
  const int64_t in_strides[] = {p.q_st, p.q_sh, p.k_st, p.k_sh, p.v_st, p.v_sh, p.k_sp, p.v_sp};
  for (int64_t sd : in_strides)
    if (sd % 8 != 0) return DLB_ERR_UNSUPPORTED;
  if (p.o_st % 4 != 0 || p.o_sh % 4 != 0) return DLB_ERR_UNSUPPORTED;
  if (B > 65535) return DLB_ERR_UNSUPPORTED;
  if (!(sm_scale > 0.0f)) return DLB_ERR_BAD_ARG;  // the tile maximum is taken before scaling

  p.Hq = Hq;
  p.Hkv = Hkv;
  p.group = Hq / Hkv;
  // workgroups are dealt round-robin to the 8 XCDs by linear id; with Hq % 8 == 0 the
  // remap in the kernel puts heads {x, x+8, ...} -> consecutive heads on one XCD so a KV
  // group's four query heads hit the same L2.
  p.xcd_heads = (Hq % 8 == 0 && Hq >= 16) ? 1 : 0;
  p.scale_log2e = sm_scale * 1.4426950408889634f;
  p.sm_scale = sm_scale;

  hipStream_t s = (hipStream_t)stream;
  const uint32_t qtiles = (uint32_t)ceil_div(max_len, kBlockM);
  if (qtiles > 65535) return DLB_ERR_UNSUPPORTED;
  const dim3 grid = dim3((uint32_t)Hq, qtiles, (uint32_t)B);
#define DLB_LAUNCH_PREFILL(DT_, D_, PG_)                                                          \
  do {                                                                                            \
    if (ragged)                                                                                   \
      hipLaunchKernelGGL((prefill_attn_kernel<DT_, D_, PG_, true>), grid, dim3(kThreads), 0, s, p);  \
    else                                                                                          \
      hipLaunchKernelGGL((prefill_attn_kernel<DT_, D_, PG_, false>), grid, dim3(kThreads), 0, s, p); \
  } while (0)
#define DLB_DISPATCH_PREFILL(PG_)                                                                \
  if (dtype == DLB_DTYPE_BF16) {                                                                 \
    if (D == 256)                                                                                \
      hipLaunchKernelGGL((prefill_attn_kernel<DLB_DTYPE_BF16, 256, PG_, true>), grid,            \
                         dim3(kThreads), 0, s, p);                                               \
    else if (D == 128) DLB_LAUNCH_PREFILL(DLB_DTYPE_BF16, 128, PG_);                              \
    else DLB_LAUNCH_PREFILL(DLB_DTYPE_BF16, 64, PG_);                                             \
  } else {                                                                                       \
    if (D == 256)                                                                                \
      hipLaunchKernelGGL((prefill_attn_kernel<DLB_DTYPE_F16, 256, PG_, true>), grid,             \
                         dim3(kThreads), 0, s, p);                                               \
    else if (D == 128) DLB_LAUNCH_PREFILL(DLB_DTYPE_F16, 128, PG_);                               \
    else DLB_LAUNCH_PREFILL(DLB_DTYPE_F16, 64, PG_);                                              \
  }
  // pages that hold whole 64-key tiles take the kernel with one page look-up per tile (the lane
  // offsets inside a page are 32-bit)
  const bool tile_pages = paged && p.page % kTileN == 0 &&
                          (int64_t)p.page * p.k_st * 2 <= 0x7fffffff && (int64_t)p.page * p.v_st * 2 <= 0x7fffffff;
  if (tile_pages) { DLB_DISPATCH_PREFILL(2) } else if (paged) { DLB_DISPATCH_PREFILL(1) } else { DLB_DISPATCH_PREFILL(0) }
#undef DLB_DISPATCH_PREFILL
#undef DLB_LAUNCH_PREFILL
  return launch_status();
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_prefill_attn_varlen(const void* q, const void* k, const void* v, void* o,
                                       const void* start_loc, const void* seq_len,
                                       int index64_mask, int B, int Hq, int Hkv, int D, int max_len, int64_t q_stride_tok,
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
  PrefillParams p = {};
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = o;
  if (index64_mask & ~3) return DLB_ERR_BAD_ARG;
  p.start_loc = idx_array(start_loc, index64_mask, 0);
  p.seq_len = idx_array(seq_len, index64_mask, 1);
  p.q_st = q_stride_tok;
  p.q_sh = q_stride_head;
  p.k_st = k_stride_tok;
  p.k_sh = k_stride_head;
  p.v_st = v_stride_tok;
  p.v_sh = v_stride_head;
  p.o_st = o_stride_tok;
  p.o_sh = o_stride_head;
  p.page = 1;
  p.page_shift = 0;
  p.window = -1;
  p.softcap = -1.0f;
  return launch_prefill(p, false, B, Hq, Hkv, D, D, max_len, sm_scale, dtype, stream);
}

extern "C" int dlb_paged_prefill_attn(const void* q, const void* k_cache, const void* v_cache,
                                      void* o, const void* block_table,
                                      const void* q_start_loc, const void* q_len,
                                      const void* kv_len, int index64_mask, int B, int Hq, int Hkv, int D,
                                      int Dv, int page, int max_blocks, int max_q_len,
                                      int64_t q_stride_tok, int64_t q_stride_head,
                                      int64_t k_stride_page, int64_t k_stride_tok,
                                      int64_t k_stride_head, int64_t v_stride_page,
                                      int64_t v_stride_tok, int64_t v_stride_head,
                                      int64_t o_stride_tok, int64_t o_stride_head,
                                      int64_t bt_stride, float sm_scale, int window_size,
                                      float logit_softcapping, int dtype, void* stream) {
  using namespace dlb;
  if (B < 0 || Hq < 1 || Hkv < 1 || D < 1 || Dv < 1 || max_q_len < 0 || page < 1 || max_blocks < 0)
    return DLB_ERR_BAD_ARG;
  if (Hq % Hkv != 0) return DLB_ERR_BAD_ARG;
  if (B == 0 || max_q_len == 0) return DLB_OK;
  if (!q || !k_cache || !v_cache || !o || !block_table || !q_start_loc || !q_len || !kv_len)
    return DLB_ERR_BAD_ARG;
  PrefillParams p = {};
  p.q = q;
  p.k = k_cache;
  p.v = v_cache;
  p.o = o;
  if (index64_mask & ~15) return DLB_ERR_BAD_ARG;
  p.block_table = idx_array(block_table, index64_mask, 0);
  p.start_loc = idx_array(q_start_loc, index64_mask, 1);
  p.seq_len = idx_array(q_len, index64_mask, 2);
  p.kv_len = idx_array(kv_len, index64_mask, 3);
  p.bt_stride = bt_stride;
  p.q_st = q_stride_tok;
  p.q_sh = q_stride_head;
  p.k_sp = k_stride_page;
  p.k_st = k_stride_tok;
  p.k_sh = k_stride_head;
  p.v_sp = v_stride_page;
  p.v_st = v_stride_tok;
  p.v_sh = v_stride_head;
  p.o_st = o_stride_tok;
  p.o_sh = o_stride_head;
  p.page = page;
  p.page_shift = (page & (page - 1)) == 0 ? __builtin_ctz((unsigned)page) : -1;
  p.window = window_size;
  p.softcap = logit_softcapping;
  return launch_prefill(p, true, B, Hq, Hkv, D, Dv, max_q_len, sm_scale, dtype, stream);
}
