// Paged decode attention for gfx950: one query token per sequence, KV cache in fixed-size
// pages addressed through a block table, grouped-query heads.
//
// Replaces the decode branch of paged_attention_fwd
// (python/dlBLAS/dlblas/kernels/paged_attention.py:604-671): _fwd_grouped_split_kernel
// (:45-234) and _reduce_split_kernel (:238-285).  Same mathematics -- per (sequence, kv head)
// the query heads of the group are batched against the head's K/V stream, online softmax in
// fp32, P rounded to the cache dtype before P.V, split-KV partials (O, m, l) combined by a
// second kernel -- with a different decomposition:
//   * the KV streams of all sequences are laid end to end (in units of 32 keys) and cut into
//     equal pieces, one per team of wavefronts (one wavefront per kv-head unit), as many
//     teams as fit on the chip at once: every wavefront streams the same number of bytes
//     whatever the mix of context lengths, instead of a fixed four-way split per sequence.
//     A piece that crosses a sequence boundary yields one partial per sequence;
//   * one wavefront per (piece, kv-head unit).  S^T = K.Q^T runs on 16x16x32 MFMA with the K rows loaded
//     straight from HBM into the A-operand layout (d is contiguous in memory and in the
//     operand), so K never touches LDS;
//   * V needs the key index contiguous per lane, so its tile is transposed on the way into
//     LDS (4 keys x 8 dims per lane, v_perm + ds_write_b64) and read back as 128-bit operands;
//     the key order inside each 32-key MFMA step is permuted so that the softmax output
//     registers ARE the B operand of O^T = V^T.P^T: P never moves between lanes.
// The kernel is an HBM stream (4 FLOP/byte at GQA 4:1); everything else is sized to keep
// tens of KB of loads in flight per CU.
#include "common.h"

namespace dlb {
namespace {

struct DecodeParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  IdxArray block_table;
  IdxArray kv_len;
  float* ws_o;      // [B, Hq, nsplit_max, D]
  float* ws_ml;     // [B, Hq, nsplit_max, 2]
  int32_t* ws_np;   // [B] partials written for each sequence
  int64_t q_sb, q_sh;
  int64_t k_sp, k_st, k_sh;
  int64_t v_sp, v_st, v_sh;
  int64_t o_sb, o_sh;
  int64_t bt_stride;
  int B, Hq, Hkv, group, hchunks;
  int page, page_shift;  // page_shift < 0: page is not a power of two
  int max_blocks;
  int min_units, nsplit_max;  // smallest piece (32-key units); partial slots per (sequence, head)
  int num_teams;
  float scale_log2e;
  float sm_scale;
  int dk, dv;      // real key / value head sizes (<= the padded size the kernel is built for)
  int window;      // > 0: keys older than (ctx - 1 - window) are masked (paged_attention.py:163-167)
  float softcap;   // > 0: logits -> softcap * tanh(logits / softcap) (paged_attention.py:186-189)
};

template <int DT>
struct Mma16;
template <>
struct Mma16<DLB_DTYPE_BF16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
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
struct Mma16<DLB_DTYPE_F16> {
  static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ unsigned int pack2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    f2 f = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, h2));
  }
};

constexpr int kTile = 64;          // keys per iteration
constexpr int kVtRowBytes = 144;   // 64 keys * 2 B + 16 B pad

// D is the padded head size the kernel is built for (64 or 128).  RAGGED: the real key size dk
// and / or value size dv is smaller (any multiple of 8): query dims past dk are zero, so whatever
// the key loads of those dims return does not count -- they are redirected to the row's first 16
// bytes to stay inside the cache -- and value dims past dv (redirected likewise) only produce
// output dims that are never stored.  The reference splits odd head sizes the same way into
// power-of-two blocks with masked loads (python/dlBLAS/dlblas/kernels/paged_attention.py:531-539).
// (The masked variant keeps a few more per-lane offsets alive: it is built for one wavefront per
// SIMD instead of two rather than spilling them.)
template <int DT, int D, bool POW2, bool RAGGED>
__global__ __launch_bounds__(64, RAGGED ? 1 : 2) void paged_decode_split_kernel(const DecodeParams p) {
  constexpr int KS = D / 32;   // MFMA k-steps over the head dim
  constexpr int MT = D / 16;   // 16-row tiles of O^T
  constexpr int DG = D / 8;    // 8-dim groups per key row

  // grid: x = (kv head, head chunk) unit, y = team.  The unit is the fastest index, so the
  // wavefronts that start together read the 256-byte head slices of the SAME token rows at the
  // same time: whole 2 KB cache rows are in flight together and DRAM pages are hit while open.
  const int unit = blockIdx.x;
  const int team = blockIdx.y;
  const int kvh = unit / p.hchunks;
  const int hchunk = unit - kvh * p.hchunks;

  const int lane = threadIdx.x & 63;
  const int g = lane >> 4;  // lane group 0..3
  const int c = lane & 15;  // column (query head) / row (key) inside a 16-tile

  __shared__ __attribute__((aligned(16))) unsigned char vt[D * kVtRowBytes];  // this wave's V^T tile
  __shared__ int32_t seg_lds[2][64];  // (first unit, units) of the 64 sequences being walked

  const unsigned short* qb = (const unsigned short*)p.q;
  const int hq_local = hchunk * 16 + c;
  const bool head_ok = hq_local < p.group;
  const int head = kvh * p.group + hq_local;

  // ---- this team's piece of the concatenated KV streams (32-key units) ----
  auto units_of = [&](int bb) { return bb < p.B ? (max(p.kv_len[bb], 0) + 31) >> 5 : 0; };
  int total = 0;
  for (int b0 = 0; b0 < p.B; b0 += 64) {
    int t = units_of(b0 + lane);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) t += __shfl_xor(t, d);
    total += t;
  }
  // (the reduction leaves the same value in every lane; say so, or every address derived from
  // it is treated as lane-dependent and the block-table lookups become vector loads that
  // share the in-order return queue of the K/V stream)
  total = __builtin_amdgcn_readfirstlane(total);
  const int upt = max((total + p.num_teams - 1) / p.num_teams, p.min_units);  // units per team
  const int lo = team * upt;
  if (lo >= total) return;
  const int hi = min(lo + upt, total);

  // one sequence segment [k_begin, k_end) of sequence b -> partial number `piece` of b
  auto process_segment = [&](int b, int k_begin, int k_end, int piece) {
  // everything that shapes the walk is wave-uniform; saying so keeps the loops and the page
  // arithmetic on the scalar unit
  b = __builtin_amdgcn_readfirstlane(b);
  const int ctx = __builtin_amdgcn_readfirstlane(p.kv_len[b]);
  k_end = __builtin_amdgcn_readfirstlane(min(k_end, ctx));
  const int kv_min = p.window > 0 ? max(ctx - 1 - p.window, 0) : 0;  // first visible key
  k_begin = __builtin_amdgcn_readfirstlane(max(k_begin, kv_min & ~31));  // the half tile holding kv_min
  const int32_t* bt = p.block_table.p + (((int64_t)b * p.bt_stride) << p.block_table.sh);
  const int bt_sh = p.block_table.sh;

  // Q^T as the B operand: lane (n = query head c, k = dims 32*ks + 8g .. +8)
  u32x4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    qf[ks] = u32x4{0u, 0u, 0u, 0u};
    if (head_ok && (!RAGGED || 32 * ks + 8 * g < p.dk))
      qf[ks] = *(const u32x4*)(qb + (int64_t)b * p.q_sb + (int64_t)head * p.q_sh + 32 * ks + 8 * g);
  }

  f32x4 o[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) o[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -__builtin_inff();
  float l_run = 0.0f;  // per-lane partial of the softmax denominator

  // Addressing: a 16-key sub-tile never straddles a page (page % 16 == 0), so its physical
  // page comes from ONE wave-uniform block-table entry (a scalar load) and every lane adds a
  // 32-bit byte offset to a uniform 64-bit base.
  const unsigned char* kbytes = (const unsigned char*)p.k + (int64_t)kvh * p.k_sh * 2;
  const unsigned char* vbytes = (const unsigned char*)p.v + (int64_t)kvh * p.v_sh * 2;
  const uint32_t k_tok_bytes = (uint32_t)p.k_st * 2u, v_tok_bytes = (uint32_t)p.v_st * 2u;
  constexpr int VL = 64 / DG < 4 ? 64 / DG : 4;  // 4-key groups of a sub-tile staged per pass
  constexpr int VPASS = 4 / VL;                  // passes per 16-key sub-tile
  const int dg = lane % DG, kgl = lane / DG;     // lanes with kgl >= VL idle (D < 128)
  // byte offsets of this lane's 16-byte pieces inside a key / value row
  uint32_t kdim_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) kdim_off[ks] = (!RAGGED || 32 * ks + 8 * g < p.dk) ? 64u * ks + 16u * g : 0u;
  const uint32_t vdim_off = (!RAGGED || 8 * dg < p.dv) ? 16u * dg : 0u;

  // The chunk is walked in half tiles of 32 keys (one k-step of the second product).  The loads
  // of half tile h + 1 are issued before half tile h is computed, so every wave keeps 16 KB of
  // requests in flight while it works; a wave's V^T staging buffer is private and LDS
  // operations of one wave execute in order, so no barrier is needed.
  struct HalfTile {
    u32x4 kf[2][KS];          // K: 2 sub-tiles of 16 keys, already in A-operand layout
    u32x4 vr[2][VPASS][4];    // V: per lane 4 consecutive keys x 8 dims per pass
  };
  // Block-table lookups are wave-uniform and must be SCALAR loads: as vector loads they sit in
  // the same in-order return queue as the K/V stream, and waiting for a page number means
  // waiting for every half tile still in flight.  The compiler will not use the scalar path for
  // memory the kernel might have written, so the load is issued by hand (and waited for on
  // the scalar counter), one half tile ahead of the loads that need the page numbers.
  int pg_ahead[2];  // physical pages of the two 16-key sub-tiles of the next half tile to load
  auto lookup_pages = [&](int h0) {
    const int32_t* entry[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int base_key = min(h0 + 16 * sub, ctx - 1);  // clamp: never look past the context
      const int pi = POW2 ? (base_key >> p.page_shift) : (base_key / p.page);
      entry[sub] = (const int32_t*)uniform_ptr((const unsigned char*)(bt + (pi << bt_sh)));
    }
    int p0, p1;
    asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(p0), "=&s"(p1)
                 : "s"(entry[0]), "s"(entry[1]));
    pg_ahead[0] = p0;
    pg_ahead[1] = p1;
  };
  auto load_half = [&](int h0, HalfTile& f) {
    const int pg_now[2] = {pg_ahead[0], pg_ahead[1]};
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int base_key = min(h0 + 16 * sub, ctx - 1);  // uniform; clamp: never read past ctx
      const int pi =
          __builtin_amdgcn_readfirstlane(POW2 ? (base_key >> p.page_shift) : (base_key / p.page));
      const int64_t pg = (int64_t)pg_now[sub];
      const int page_key0 = pi * p.page;
      {
        const int key = min(h0 + 16 * sub + c, ctx - 1);
        const unsigned char* base = kbytes + pg * p.k_sp * 2;
        // K rows are read as two half-line (64-byte) pieces by consecutive k-steps: keep them
        // cacheable so the second piece hits the line the first one brought in
        const uint32_t off = (uint32_t)(key - page_key0) * k_tok_bytes;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (RAGGED) f.kf[sub][ks] = *(const u32x4*)(base + off + kdim_off[ks]);
          else f.kf[sub][ks] = *(const u32x4*)(base + off + 16u * g + 64 * ks);
        }
      }
      {
        const unsigned char* base = vbytes + pg * p.v_sp * 2;
#pragma unroll
        for (int ps = 0; ps < VPASS; ++ps) {
          const int key0 = min(h0 + 16 * sub + 4 * (ps * VL + kgl), ctx - 1);
          const int room = ctx - 1 - key0;
          if (kgl < VL) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const uint32_t off = (uint32_t)(key0 - page_key0 + min(r, room)) * v_tok_bytes + vdim_off;
              f.vr[sub][ps][r] = __builtin_nontemporal_load((const u32x4*)(base + off));
            }
          }
        }
      }
    }
    lookup_pages(h0 + 32);
  };
  // st = parity of the half tile inside its 64-key tile = which 4 units of a V^T row it uses
  auto compute_half = [&](int h0, const HalfTile& f, int st) {
    // ---- S^T = K . Q^T (rows = keys, cols = query heads) ----
    f32x4 s[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      s[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) s[sub] = Mma16<DT>::run(f.kf[sub][ks], qf[ks], s[sub]);
    }

    // ---- V^T into LDS: Vt[d][pos], pos = 32*st + 8*g' + 4*a + r for key 32*st + 16*a + 4*g' + r
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int ps = 0; ps < VPASS; ++ps) {
        if (kgl < VL) {
          const int unit = 4 * st + ps * VL + kgl;  // 16-byte unit inside the row
          const int half = sub;                     // 8-byte half inside the unit
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            const u32x4* v4 = f.vr[sub][ps];
            const unsigned int lo01 = __builtin_amdgcn_perm(v4[1][w], v4[0][w], 0x05040100u);
            const unsigned int lo23 = __builtin_amdgcn_perm(v4[3][w], v4[2][w], 0x05040100u);
            const unsigned int hi01 = __builtin_amdgcn_perm(v4[1][w], v4[0][w], 0x07060302u);
            const unsigned int hi23 = __builtin_amdgcn_perm(v4[3][w], v4[2][w], 0x07060302u);
            const int d0 = 8 * dg + 2 * w;
            const int sw = ((d0 >> 4) & 3) << 1;  // same for d0 and d0 + 1
            unsigned char* row = vt + d0 * kVtRowBytes + ((unit ^ sw) << 4) + (half << 3);
            *(u32x2*)(row) = u32x2{lo01, lo23};
            *(u32x2*)(row + kVtRowBytes) = u32x2{hi01, hi23};
          }
        }
      }
    }

    // ---- online softmax over these 32 keys (log2 domain) ----
    float mloc = -__builtin_inff();
    if (p.softcap > 0.0f) {  // one uniform branch for the half tile, not one per element
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          s[sub][i] = p.softcap * tanhf(s[sub][i] * p.sm_scale / p.softcap) * 1.4426950408889634f;
    } else {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[sub][i] *= p.scale_log2e;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = h0 + 16 * sub + 4 * g + i;
        const float x = (key < k_end && key >= kv_min) ? s[sub][i] : -__builtin_inff();
        s[sub][i] = x;
        mloc = fmaxf(mloc, x);
      }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    const float m_new = fmaxf(m_run, mloc);
    // a half tile can be entirely masked (sliding window, chunk tail): keep exponents finite
    const float m_ref = (m_new == -__builtin_inff()) ? 0.0f : m_new;
    if (__any(m_new > m_run)) {  // wave-uniform: skip the rescale when no maximum moved
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
      l_run *= alpha;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
    }
    m_run = m_new;
    float psum = 0.0f;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = __builtin_amdgcn_exp2f(s[sub][i] - m_ref);
        s[sub][i] = e;
        psum += e;
      }
    }
    l_run += psum;

    // P^T as the B operand: slots 0..3 <- sub-tile 0, slots 4..7 <- sub-tile 1
    u32x4 pf;
    pf[0] = Mma16<DT>::pack2(s[0][0], s[0][1]);
    pf[1] = Mma16<DT>::pack2(s[0][2], s[0][3]);
    pf[2] = Mma16<DT>::pack2(s[1][0], s[1][1]);
    pf[3] = Mma16<DT>::pack2(s[1][2], s[1][3]);

    // ---- O^T += V^T . P^T ----
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int d = 16 * mt + c;
      const int sw = (mt & 3) << 1;
      const u32x4 a = *(const u32x4*)(vt + d * kVtRowBytes + (((4 * st + g) ^ sw) << 4));
      o[mt] = Mma16<DT>::run(a, pf, o[mt]);
    }
  };

  HalfTile ha, hb;
  if (k_begin < k_end) {  // (a segment entirely before the window is empty)
    lookup_pages(k_begin);
    load_half(k_begin, ha);
    int t0 = k_begin;
    // steady state: the tile has both halves and another tile follows.  No run-time condition
    // surrounds a load here: where the two paths of a branch around loads join, the compiler
    // has to wait as if the loads had not been issued, i.e. for the ones just sent.
    for (; t0 + kTile < k_end; t0 += kTile) {
      load_half(t0 + 32, hb);
      __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the arithmetic below
      compute_half(t0, ha, 0);
      __builtin_amdgcn_sched_barrier(0);
      load_half(t0 + kTile, ha);
      __builtin_amdgcn_sched_barrier(0);
      compute_half(t0 + 32, hb, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    // last tile: one or two halves
    const bool second = t0 + 32 < k_end;
    if (second) load_half(t0 + 32, hb);
    __builtin_amdgcn_sched_barrier(0);
    compute_half(t0, ha, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (second) compute_half(t0 + 32, hb, 1);
  }

  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);

  if (head_ok) {
    const int64_t slot = ((int64_t)b * p.Hq + head) * p.nsplit_max + piece;
    float* wo = p.ws_o + slot * D;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(f32x4*)(wo + 16 * mt + 4 * g) = o[mt];
    if (g == 0) {
      p.ws_ml[slot * 2 + 0] = m_run;  // -inf with l = 0 for an empty segment: weight 0 in the combine
      p.ws_ml[slot * 2 + 1] = l_run;
    }
  }
  };  // process_segment

  // ---- walk the sequences this piece overlaps ----
  int carry = 0;  // units of all sequences before b0
  for (int b0 = 0; b0 < p.B; b0 += 64) {
    const int t = units_of(b0 + lane);
    const int incl = wave_inclusive_scan(t);
    const int excl = carry + incl - t;
    uint64_t hit = __ballot(t > 0 && excl < hi && excl + t > lo);
    // park the per-sequence values in LDS: nothing per-lane stays live across a segment
    seg_lds[0][lane] = excl;
    seg_lds[1][lane] = t;
    carry = __builtin_amdgcn_readfirstlane(carry + __shfl(incl, 63));
    while (hit) {  // wave-uniform
      const int l = __builtin_ctzll(hit);
      hit &= hit - 1;
      const int b = b0 + l;
      const int pb = __builtin_amdgcn_readfirstlane(seg_lds[0][l]);
      const int tb = __builtin_amdgcn_readfirstlane(seg_lds[1][l]);
      const int first_team = pb / upt;
      if (team == first_team && unit == 0 && lane == 0)
        p.ws_np[b] = (pb + tb - 1) / upt - first_team + 1;
      process_segment(b, (max(lo, pb) - pb) * 32, (min(hi, pb + tb) - pb) * 32, team - first_team);
    }
    if (carry >= hi) break;
  }
}

// Combine the partials of one (sequence, head): O = sum_s 2^(m_s - m) O_s / sum_s 2^(m_s - m) l_s
// (paged_attention.py:238-285 with the exponent in base 2).  Lane s of every wave fetches
// (m_s, l_s) so the weights come from two wave reductions; the O_s rows are then read with all
// loads of a group of four in flight.
template <int DT, int D>
__global__ __launch_bounds__(D) void paged_decode_combine_kernel(const DecodeParams p) {
  const int head = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int lane = d & 63;
  const int ctx = p.kv_len[b];
  float acc = 0.0f;
  if (ctx > 0) {
    const int ns = p.ws_np[b];  // pieces of this sequence (empty ones carry m = -inf, l = 0)
    const int64_t slot0 = ((int64_t)b * p.Hq + head) * p.nsplit_max;
    float m = -__builtin_inff();
    for (int s0 = 0; s0 < ns; s0 += 64) {
      float ms = (s0 + lane < ns) ? p.ws_ml[(slot0 + s0 + lane) * 2] : -__builtin_inff();
#pragma unroll
      for (int x = 32; x >= 1; x >>= 1) ms = fmaxf(ms, __shfl_xor(ms, x));
      m = fmaxf(m, ms);
    }
    float den = 0.0f;
    for (int s0 = 0; s0 < ns; s0 += 64) {
      const bool live = s0 + lane < ns;
      const float w = live ? __builtin_amdgcn_exp2f(p.ws_ml[(slot0 + s0 + lane) * 2] - m) : 0.0f;
      float wl = live ? w * p.ws_ml[(slot0 + s0 + lane) * 2 + 1] : 0.0f;
#pragma unroll
      for (int x = 32; x >= 1; x >>= 1) wl += __shfl_xor(wl, x);
      den += wl;
      const int n = min(64, ns - s0);
      for (int s = 0; s < n; s += 4) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = (s + u < n) ? p.ws_o[(slot0 + s0 + s + u) * D + d] : 0.0f;
#pragma unroll
        for (int u = 0; u < 4; ++u) acc += __shfl(w, min(s + u, 63)) * v[u];
      }
    }
    acc /= den;
  }
  if (d < p.dv) Elem<DT>::store1(p.o, (int64_t)b * p.o_sb + (int64_t)head * p.o_sh + d, acc);
}

// smallest piece a team may get, in 32-key units: 512 keys, less for small problems so that
// the chip still sees a few thousand wavefronts
int pick_min_units(int B, int Hkv, int hchunks, int max_ctx) {
  const int64_t units = (int64_t)B * Hkv * hchunks;
  int kps = 512;
  while (kps > 128 && units * ((max_ctx + kps - 1) / kps) < 4096) kps >>= 1;
  return kps / 32;
}

// partial slots per (sequence, head): a sequence of T units cut into pieces of >= min_units
// overlaps at most T / min_units + 2 of them
int partial_slots(int max_ctx, int min_units) {
  const int t = (max_ctx + 31) / 32;
  return t / min_units + 2;
}

// teams that are resident together: 8 wavefronts per CU (2 per SIMD) / wavefronts per team
int pick_num_teams(int units_per_team) {
  return max(1, current_device_cu_count() * 8 / units_per_team);
}

}  // namespace
}  // namespace dlb

extern "C" size_t dlb_paged_decode_ws_bytes(int B, int Hq, int Hkv, int D, int page,
                                            int max_blocks) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || D > 256 || page <= 0 || max_blocks <= 0) return 0;
  D = D <= 64 ? 64 : D <= 128 ? 128 : 256;  // the head size the kernels are built for
  const int group = Hq / Hkv;
  const int hchunks = (group + 15) / 16;
  const int64_t max_ctx = (int64_t)page * max_blocks;
  if (max_ctx > 0x7fffffff) return 0;
  const int64_t ns = dlb::partial_slots((int)max_ctx, dlb::pick_min_units(B, Hkv, hchunks, (int)max_ctx));
  return (size_t)B * Hq * ns * (D + 2) * sizeof(float) + (size_t)B * sizeof(int32_t);
}

extern "C" int dlb_paged_decode_attn(const void* q, const void* k_cache, const void* v_cache,
                                     void* o, const void* block_table, const void* kv_len,
                                     int index64_mask, int B, int Hq, int Hkv, int D, int Dv, int page,
                                     int max_blocks, int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_page,
                                     int64_t k_stride_tok, int64_t k_stride_head,
                                     int64_t v_stride_page, int64_t v_stride_tok,
                                     int64_t v_stride_head, int64_t o_stride_b, int64_t o_stride_h,
                                     int64_t bt_stride, float sm_scale, int window_size,
                                     float logit_softcapping, int dtype, void* ws,
                                     size_t ws_bytes, void* stream) {
  using namespace dlb;
  if (B < 0 || Hq < 1 || Hkv < 1 || D < 1 || Dv < 1 || page < 1 || max_blocks < 1) return DLB_ERR_BAD_ARG;
  if (Hq % Hkv != 0) return DLB_ERR_BAD_ARG;
  if (B == 0) return DLB_OK;
  if (!q || !k_cache || !v_cache || !o || !block_table || !kv_len) return DLB_ERR_BAD_ARG;
  if (D % 8 != 0 || Dv % 8 != 0 || D > 256 || Dv > 256) return DLB_ERR_UNSUPPORTED;
  // head size the kernel instance is built for; past 128 one instance, for 256, takes every size
  // on its ragged path
  const int Dp = (D <= 64 && Dv <= 64) ? 64 : (D <= 128 && Dv <= 128) ? 128 : 256;
  const bool ragged = D != Dp || Dv != Dp || Dp == 256;
  if (page % 16 != 0) return DLB_ERR_UNSUPPORTED;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
  if ((int64_t)page * max_blocks > 0x7fffffff) return DLB_ERR_UNSUPPORTED;
  // per-lane byte offsets inside a page are 32-bit
  if ((int64_t)page * k_stride_tok * 2 > 0x7fffffff || (int64_t)page * v_stride_tok * 2 > 0x7fffffff)
    return DLB_ERR_UNSUPPORTED;
  // 128-bit operand loads
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) return DLB_ERR_UNSUPPORTED;
  const int64_t strides[] = {q_stride_b,   q_stride_h,    k_stride_page, k_stride_tok,
                             k_stride_head, v_stride_page, v_stride_tok,  v_stride_head};
  for (int64_t sd : strides)
    if (sd % 8 != 0) return DLB_ERR_UNSUPPORTED;
  const size_t need = dlb_paged_decode_ws_bytes(B, Hq, Hkv, Dp, page, max_blocks);
  if (!ws || ws_bytes < need) return DLB_ERR_WORKSPACE;

  DecodeParams p;
  p.q = q;
  p.k = k_cache;
  p.v = v_cache;
  p.o = o;
  if (index64_mask & ~3) return DLB_ERR_BAD_ARG;
  p.block_table = idx_array(block_table, index64_mask, 0);
  p.kv_len = idx_array(kv_len, index64_mask, 1);
  p.q_sb = q_stride_b;
  p.q_sh = q_stride_h;
  p.k_sp = k_stride_page;
  p.k_st = k_stride_tok;
  p.k_sh = k_stride_head;
  p.v_sp = v_stride_page;
  p.v_st = v_stride_tok;
  p.v_sh = v_stride_head;
  p.o_sb = o_stride_b;
  p.o_sh = o_stride_h;
  p.bt_stride = bt_stride;
  p.B = B;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.group = Hq / Hkv;
  p.hchunks = (p.group + 15) / 16;
  p.page = page;
  p.page_shift = -1;
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == page) p.page_shift = sh;
  p.max_blocks = max_blocks;
  const int max_ctx = page * max_blocks;
  p.min_units = pick_min_units(B, Hkv, p.hchunks, max_ctx);
  p.nsplit_max = partial_slots(max_ctx, p.min_units);
  p.scale_log2e = sm_scale * 1.4426950408889634f;
  p.sm_scale = sm_scale;
  p.window = window_size;
  p.softcap = logit_softcapping;
  p.dk = D;
  p.dv = Dv;
  p.ws_o = (float*)ws;
  p.ws_ml = p.ws_o + (size_t)B * Hq * p.nsplit_max * Dp;
  p.ws_np = (int32_t*)(p.ws_ml + (size_t)B * Hq * p.nsplit_max * 2);

  hipStream_t s = (hipStream_t)stream;
  const int units = Hkv * p.hchunks;
  p.num_teams = pick_num_teams(units);
  if (units > 65535 || p.num_teams > 65535) return DLB_ERR_UNSUPPORTED;
  const dim3 grid1((uint32_t)units, (uint32_t)p.num_teams);
  const dim3 grid2((uint32_t)Hq, (uint32_t)B);
#define DLB_LAUNCH_SPLIT(DT_, D_, P2_, RG_) \
  hipLaunchKernelGGL((paged_decode_split_kernel<DT_, D_, P2_, RG_>), grid1, dim3(64), 0, s, p)
#define DLB_LAUNCH_DECODE(DT_, D_)                                                        \
  do {                                                                                    \
    if (p.page_shift >= 0) {                                                              \
      if (ragged) DLB_LAUNCH_SPLIT(DT_, D_, true, true);                                  \
      else DLB_LAUNCH_SPLIT(DT_, D_, true, false);                                        \
    } else {                                                                              \
      if (ragged) DLB_LAUNCH_SPLIT(DT_, D_, false, true);                                 \
      else DLB_LAUNCH_SPLIT(DT_, D_, false, false);                                       \
    }                                                                                     \
    hipLaunchKernelGGL((paged_decode_combine_kernel<DT_, D_>), grid2, dim3(D_), 0, s, p); \
  } while (0)
#define DLB_LAUNCH_DECODE_256(DT_)                                                         \
  do {                                                                                    \
    if (p.page_shift >= 0) DLB_LAUNCH_SPLIT(DT_, 256, true, true);                        \
    else DLB_LAUNCH_SPLIT(DT_, 256, false, true);                                         \
    hipLaunchKernelGGL((paged_decode_combine_kernel<DT_, 256>), grid2, dim3(256), 0, s, p); \
  } while (0)
  if (dtype == DLB_DTYPE_BF16) {
    if (Dp == 256) DLB_LAUNCH_DECODE_256(DLB_DTYPE_BF16);
    else if (Dp == 128) DLB_LAUNCH_DECODE(DLB_DTYPE_BF16, 128);
    else DLB_LAUNCH_DECODE(DLB_DTYPE_BF16, 64);
  } else {
    if (Dp == 256) DLB_LAUNCH_DECODE_256(DLB_DTYPE_F16);
    else if (Dp == 128) DLB_LAUNCH_DECODE(DLB_DTYPE_F16, 128);
    else DLB_LAUNCH_DECODE(DLB_DTYPE_F16, 64);
  }
#undef DLB_LAUNCH_DECODE_256
#undef DLB_LAUNCH_SPLIT
#undef DLB_LAUNCH_DECODE
  return launch_status();
}
