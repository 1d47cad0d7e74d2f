// fp8 (OCP e4m3fn) fused-MoE building blocks for gfx950:
//   * per-token-group activation quantisation (groups of 128 along K, fp32 scales);
//   * expert-grouped GEMM over block-aligned routing (blocks of 64 or 128 rows, one expert per
//     block) on the 32x32x64 f8f6f4 MFMA, with the block scales of every 128-deep K chunk
//         out = sum_kc mfma(x_q[:, kc], w_q[:, kc]) * x_scale[row, kc] * w_scale[n / 128, kc]
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
// fused_moe, with 32x32x16 MFMAs and no scales.
//
// GEMM mapping.  The MFMA runs "transposed": weight rows are the A operand (M index = output
// column n), activations the B operand (N index = token row), so a lane's sixteen accumulator
// registers of a 32x32 tile are 4 x 4 consecutive n of ONE token: the activation scale is a
// per-lane scalar and the epilogues store runs of adjacent outputs.  Weight fragments go
// straight from HBM/L2 into operand registers (each wave owns its own n range, so nothing is
// shared between waves); only the 128 x 128-byte activation chunk passes through LDS.
#include <type_traits>

#include "common.h"
#include "quant_fp8.h"

namespace dlb {
namespace {

// K chunks of 128 bytes whose block scales the fp8 grouped GEMM parks in LDS: reduction lengths
// up to 128 * 128 = 16384 (checked on the host before the launch)
constexpr int kMoeMaxKChunks = 128;
// Floors of the scales inside the fp8 GEMM.  The accumulators are kept relative to the scale of
// the current K chunk (multiplied by s(k) / s(k + 1) between chunks), so |sum| / s(k) must stay
// inside fp32: with the activation scale floored just below the smallest value the quantiser
// itself produces (1e-10 / 448 = 2.2e-13, the scale of an all-zero group) and the weight block
// scale floored at 1e-12 (a block whose values are below 4.5e-10), a row may mix empty groups,
// empty weight blocks and groups of any realistic magnitude without leaving the fp32 range.
constexpr float kActScaleFloor = 1e-13f;
constexpr float kWScaleFloor = 1e-12f;

// ---------------------------------------------------------------------------------------
// per-token-group quantisation (the body lives in quant_fp8.h)
// ---------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kQuantThreads) void quant_fp8_group128_kernel(const QuantParams q) {
  quant_fp8_group128_block<DT>(q, blockIdx.x);
}

// ---------------------------------------------------------------------------------------
// grouped GEMM
// ---------------------------------------------------------------------------------------
struct MoeGemmParams {
  const unsigned char* a;     // activations fp8 [rows, K] (or 16-bit: K = bytes per row)
  const float* a_scale;       // [rows, K / 128]
  const unsigned char* w;     // weights [E_local, N, K]
  const float* w_scale;       // [E_local, N / 128, K / 128]
  IdxArray sorted_ids;        // [num_mblocks * block_m] routing slots grouped by expert
  IdxArray counts;            // [num_experts] routed slots per (global) expert
  // launcher form of the routing (non-gated kernel only): the slot list is NOT padded per expert;
  // expert e owns its positions seg_start[e] .. counts[e] - 1 (counts then holds the segment ENDS)
  IdxArray seg_start;         // p == nullptr: block-aligned list
  int64_t a_rows;             // rows of `a` when it is read in sorted order (reads are clamped to it)
  int gather_a;               // non-gated kernel: rows of `a` are gathered by token (slot / topk)
  int scatter_c;              // non-gated kernel: output row = routing slot (else the sorted position)
  int num_experts;            // global expert count = length of counts
  int num_mblocks;            // capacity of sorted_ids in blocks
  int bm_shift;               // log2(block_m): 6 or 7
  int num_ntiles;
  int K, N, KC;               // K = bytes per activation / weight row, KC = K / 128
  int topk, numel;            // flat slots = tokens * topk (also the pad sentinel)
  int num_tokens;
  int expert_offset;          // weights hold experts [expert_offset, expert_offset + E_local)
  int num_local;              // E_local
  // gate_up flavour
  unsigned char* hq;          // [num_mblocks * block_m, I] fp8, or 16-bit when QT = 1
  float* hs;                  // [num_mblocks * block_m, I / 128]
  int I;
  // down flavour
  void* out;                  // [numel, N] bf16/f16
  const float* topk_w;        // [numel]
};

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

// One weight unit = the lane's operand pieces of one 64-byte half (HK) of a 128-byte K chunk for
// the wave's two column tiles: 2 tiles x 2 pieces of 16 bytes, uniform base + 32-bit lane
// offsets.  WL 1 (operand order): the half's pieces sit 512 bytes apart in the tile's 2 KB
// block; WL 0 (row-major): 32 bytes apart in the weight row.  Plain loads: the compiler owns
// these registers and places the waits for them itself.
template <int WL, int HK>
__device__ __forceinline__ void load_w_unit(u32x4 (&b)[2][2], unsigned int voff0, unsigned int voff1,
                                            const unsigned char* sbase) {
  typedef const __attribute__((address_space(1))) unsigned char* gptr_t;
  typedef const __attribute__((address_space(1))) u32x4* gvec_t;
  constexpr int o0 = WL ? HK * 1024 : HK * 64;
  constexpr int o1 = WL ? HK * 1024 + 512 : HK * 64 + 32;
  gptr_t g = (gptr_t)sbase;  // wave-uniform base, 32-bit lane offsets
  b[0][0] = *(gvec_t)(g + (uint64_t)voff0 + o0);
  b[0][1] = *(gvec_t)(g + (uint64_t)voff0 + o1);
  b[1][0] = *(gvec_t)(g + (uint64_t)voff1 + o0);
  b[1][1] = *(gvec_t)(g + (uint64_t)voff1 + o1);
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// ---- which tile does this workgroup compute? ------------------------------------------------
// Tiles are numbered expert by expert (local experts only), inside an expert column tile by
// column tile, and inside a column tile row block by row block -- so tiles that follow each
// other share their weights.  Workgroup ids are dealt round-robin to the 8 XCDs; XCD x takes the
// x-th eighth of that order and its workgroups take consecutive tiles of it in the order the
// dispatcher starts them.  At any moment an XCD therefore works on a handful of experts: an
// expert's weights are streamed once while its few row blocks run side by side, and its
// activation rows stay in that XCD's L2 across all its column tiles.
// The expert's first block and its row count come from the per-expert counts of the alignment
// (block b of expert e starts at sum_{e' < e} ceil(count / block_m) + b): one load per lane
// and two wave scans.  All results are wave-uniform.
struct TileId {
  int e;     // local expert
  int row0;  // first position of the tile's rows in sorted_ids
  int nt;    // column tile
  int rows;  // real (unpadded) rows of the block, 1 .. block_m
};
__device__ __forceinline__ bool find_tile(const MoeGemmParams& p, int lane, TileId& t) {
  const int bm = 1 << p.bm_shift;
  const bool segs = p.seg_start.p != nullptr;
  int cnt[4], nb[4], tl[4], st[4];
  int nb_sum = 0, tl_sum = 0;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int e = 4 * lane + c;
    st[c] = (segs && e < p.num_experts) ? p.seg_start[e] : 0;
    cnt[c] = e < p.num_experts ? max(p.counts[e] - st[c], 0) : 0;
    nb[c] = (cnt[c] + bm - 1) >> p.bm_shift;
    const bool local = e >= p.expert_offset && e < p.expert_offset + p.num_local;
    tl[c] = local ? nb[c] * p.num_ntiles : 0;
    nb_sum += nb[c];
    tl_sum += tl[c];
  }
  const int nb_incl = wave_inclusive_scan(nb_sum);
  const int tl_incl = wave_inclusive_scan(tl_sum);
  const int total = __builtin_amdgcn_readlane(tl_incl, 63);
  const int per_xcd = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, i = blockIdx.x >> 3;
  const int logical = xcd * per_xcd + i;
  if (i >= per_xcd || logical >= total) return false;
  const unsigned long long hit = __ballot(tl_incl > logical);
  const int L = __builtin_ctzll(hit);  // the lane whose four experts hold the tile
  int rem = logical - __builtin_amdgcn_readlane(tl_incl - tl_sum, L);
  int mbase = __builtin_amdgcn_readlane(nb_incl - nb_sum, L);
  int e = 4 * L, nbe = 1, ce = 0, se = 0;
  bool found = false;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int tc = __builtin_amdgcn_readlane(tl[c], L);
    const int nc = __builtin_amdgcn_readlane(nb[c], L);
    const int cc = __builtin_amdgcn_readlane(cnt[c], L);
    const int sc = __builtin_amdgcn_readlane(st[c], L);
    if (!found) {
      if (rem < tc) {
        found = true;
        e = 4 * L + c;
        nbe = nc;
        ce = cc;
        se = sc;
      } else {
        rem -= tc;
        mbase += nc;
      }
    }
  }
  const int nt = rem / nbe;
  const int rb = rem - nt * nbe;
  t.e = e - p.expert_offset;
  // block-aligned list: block mbase + rb; launcher form: the expert's own segment
  t.row0 = segs ? se + (rb << p.bm_shift) : (mbase + rb) << p.bm_shift;
  t.nt = nt;
  t.rows = min(bm, ce - (rb << p.bm_shift));
  // (counts that do not fit the slot list: touch nothing)
  return segs ? t.row0 + t.rows <= p.numel : (mbase + rb) < p.num_mblocks;
}

// QT = 0: fp8 operands with block scales; QT = 1: 16-bit operands of type DT, no scales.
// GATED = true : gate_up GEMM (N = 2I), tile = 128 gate cols + the matching 128 up cols,
//                epilogue silu(gate) * up -> fp8 + per-128 scale, rows kept in sorted order.
// GATED = false: down GEMM, tile = 256 cols, epilogue * routing weight -> out[slot, n].
// WL = weight layout (0 row-major, 1 operand order).
//
// Tile = one alignment block (up to 128 routing slots = four 32-row tiles) x 256 output columns,
// four waves, two workgroups per CU.  A wave owns 64 output columns (two 32-column tiles; gated:
// 32 gate + the matching 32 up columns) x all the rows: 4 x 2 accumulator tiles of the 32x32x64
// (fp8) / 32x32x16 (16 bit) MFMA.  Lane (j = lane % 32, h = lane / 32) supplies, for weight
// row / token j, the four 16-byte pieces q = 0..3 of a 128-byte K chunk at chunk offset
// 32 q + 16 h; the fp8 MFMA of chunk half m consumes pieces 2m and 2m + 1, the 16-bit MFMA q
// consumes piece q.  Its 16 accumulators of a tile are token j, columns 8 (r / 4) + 4 h + r % 4.
// Row tiles made of padding only are skipped (wave-uniform), so the matrix work follows the
// routed rows in steps of 32.
//
// Block scales without a second accumulator.  The MFMAs accumulate in place; between two
// chunks an accumulator tile is multiplied by s(k) / s(k + 1), s(k) = x_scale[row, k] *
// w_scale[n / 128, k], so that it always holds sum_{k' <= k} P(k') s(k') / s(k), and the
// epilogue multiplies by the last s.  One multiply per accumulator and chunk, as many vector
// operations as acc += P * s would take, but no separate product tile: 128 accumulators, two
// chunks of weights and two fragment buffers fit the 256 registers of a wave at two waves per
// SIMD.  (Scales are floored -- kActScaleFloor, kWScaleFloor -- so that a zero scale cannot
// divide and the ratio of two neighbouring chunks cannot push an accumulator out of fp32.)
//
// Data movement:
//   * weights: global -> operand registers with plain loads, in units of (chunk half, both
//     column tiles) = 4 x 16 bytes per lane; two chunks of units live in registers, each unit
//     re-loaded right after its last use for the chunk after next (1.5 chunks ahead).  The
//     compiler owns these registers and places their waits (issued from inline assembly the
//     four pieces of a unit do not end up in adjacent registers, and the copies that gather
//     them cost more than the exact waits save);
//   * activations: global -> LDS directly, by hand (three chunk slots of 128 x 128 bytes, rows
//     swizzled by (row >> 1) & 7 in 16-byte pieces), wave w stages row tile w, issued two chunks
//     ahead; one barrier per chunk, between its two halves, publishes the next chunk; the
//     activation scales of a chunk travel with it (one 4-byte copy per wave).  The compiler does
//     not see these copies, so the kernel waits for them itself with a constant vmcnt: every
//     wave issues the same number of vector-memory operations per chunk (chunks past K re-load
//     clamped addresses, waves whose row tile is padding copy one dummy line);
//   * the block scales of the wave's two column tiles are parked in LDS once per tile.
// None of this may go through scratch memory: the build checks that the kernel spills nothing.
template <bool GATED, int DT, int QT, int WL>
__global__ __launch_bounds__(256, 2) void moe_gemm_kernel(const MoeGemmParams p) {
  constexpr int NX = 3;                 // activation chunk slots in LDS
  constexpr int kXSlot = 128 * 128;     // bytes of one slot
  constexpr int kScWave = 128;          // scale strip of a wave per slot: its 32 activation scales
  constexpr int kMaxKC = kMoeMaxKChunks;  // chunks of block scales parked in LDS (K <= 16384 bytes)
  constexpr int kScSlot = 4 * kScWave;
  constexpr int D = QT == 0 ? 5 : 4;    // direct-to-LDS operations per wave and chunk
  __shared__ __attribute__((aligned(1024))) unsigned char x_lds[NX * kXSlot];
  __shared__ __attribute__((aligned(16))) unsigned char sc_lds[NX * kScSlot];
  __shared__ float ws_lds[4][2][kMaxKC];  // block scales of wave w's column tile ct, by chunk
  __shared__ float red_lds[4][128];
  __shared__ int32_t sid_lds[128];
  __shared__ float rw_lds[128];
  __shared__ __attribute__((aligned(16))) uint32_t xoff_lds[256][4];  // copy source offsets per lane

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int h = lane >> 5;
  const int j = lane & 31;
  const int drow = lane >> 3, dpc = lane & 7;

  TileId tile;
  if (!find_tile(p, lane, tile)) return;
  // The rest of the kernel exists twice, for tiles of four and of two 32-row tiles (blocks with
  // more / at most 64 real rows), each with its loops fully unrolled: row tiles of padding are
  // skipped at that granularity without a run-time condition inside the main loop, and the two
  // versions share no live values (each ends the kernel), so neither costs the other registers.
  auto run = [&](auto nrt_tag) {
  constexpr int NRT = decltype(nrt_tag)::value;
  const int e = tile.e, nt = tile.nt;
  const int nrt_real = (tile.rows + 31) >> 5;  // row tiles that hold real rows (<= NRT)
  const int row0 = tile.row0;
  const int K = p.K, KC = p.KC;
  const bool stager = wave < nrt_real;  // this wave's row tile is real: it stages those rows

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
  // weight unit (chunk kc, half HK); past the end the last chunk is read again
  auto issue_w = [&](auto hk, int kc, u32x4 (&b)[2][2]) {
    const unsigned char* sbase = uniform_ptr(wbase + min(kc, KC - 1) * kWChunk);
    load_w_unit<WL, decltype(hk)::value>(b, woff[0], woff[1], sbase);
  };
  using H0 = std::integral_constant<int, 0>;
  using H1 = std::integral_constant<int, 1>;

  u32x4 wr[2][2][2][2];  // weight units [chunk parity][chunk half][column tile][piece]
  // the first unit goes out before the routing slots are even known: it only needs the expert
  issue_w(H0{}, 0, wr[0][0]);

  // ---- routing slots.  Gated: the rows this lane stages (four) and the row whose scale it
  // fetches.  Down: thread t < 128 keeps slot and routing weight of row t for the epilogue.
  int sid_x[4] = {0, 0, 0, 0};
  int sid_s = 0;
  // (positions past the tile's real rows hold the pad sentinel in a block-aligned list and another
  // expert's slots in the launcher form: they are not read)
  auto slot_at = [&](int r) -> int { return r < tile.rows ? p.sorted_ids[row0 + r] : p.numel; };
  const bool gather = GATED || p.gather_a;
  if (gather && stager) {
#pragma unroll
    for (int i = 0; i < 4; ++i) sid_x[i] = slot_at(32 * wave + 8 * i + drow);
    if (QT == 0) sid_s = slot_at(32 * wave + j);
  }
  if (!GATED) {
    if (tid < 128) {
      // destination row of the tile's row `tid` (-1: none) and its routing weight
      int dst = -1;
      float rwt = 0.0f;
      if (tid < tile.rows) {
        const int sid = p.sorted_ids[row0 + tid];
        if (sid >= 0 && sid < p.numel) {
          dst = p.scatter_c ? sid : row0 + tid;
          rwt = p.topk_w ? p.topk_w[sid] : 1.0f;
        }
      }
      sid_lds[tid] = dst;  // published by the barrier that opens the main loop
      rw_lds[tid] = rwt;
    }
  }
  // source row of the tile's row r whose routing slot is sid (gated: the slot's token; pad
  // slots read a valid row)
  auto src_row_of = [&](int sid, int r) -> uint32_t {
    if (gather) return (uint32_t)min(max(sid, 0) / p.topk, p.num_tokens - 1);
    return (uint32_t)min((int64_t)(row0 + r), p.a_rows - 1);
  };
  // ---- activation staging: per chunk 16 instructions of 8 rows x 128 bytes, four per wave
  // (its own row tile); lane -> (row, physical piece), the logical piece it fetches undoes the
  // swizzle.  A wave whose row tile is padding copies the same 16 bytes with every lane.
  // (the four byte offsets of a lane are parked in LDS and re-read for every chunk: they would
  // otherwise occupy four registers for the whole kernel)
  {
    u32x4 xo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 32 * wave + 8 * i + drow;
      xo[i] = stager ? src_row_of(sid_x[i], r) * (uint32_t)K + (uint32_t)((dpc ^ ((r >> 1) & 7)) << 4) : 0u;
    }
    *(u32x4*)xoff_lds[tid] = xo;  // read back by the same lane only: no barrier needed
  }
  // activation scales: one 4-byte copy per wave and chunk with 32 lanes active, lane l fetching
  // the scale of the wave's staging row l.  The block scales of the wave's two column tiles for
  // all chunks are fetched once, here, and parked in LDS.
  uint32_t sc_voff = 0;
  if (QT == 0) {
    if (stager && lane < 32) sc_voff = src_row_of(sid_s, 32 * wave + j) * (uint32_t)KC * 4u;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const int sblk = min(ncol[ct] >> 7, (p.N >> 7) - 1);
      const float* src = p.w_scale + ((int64_t)e * (p.N >> 7) + sblk) * KC;
#pragma unroll
      for (int i = 0; i < kMaxKC / 64; ++i) {
        const int kc = lane + 64 * i;
        if (kc < KC) ws_lds[wave][ct][kc] = src[kc];
      }
    }
  }

  const unsigned int x_dst0 = lds_addr(x_lds) + wave * 4096;
  const unsigned int sc_dst0 = lds_addr(sc_lds) + wave * kScWave;
  // all direct-to-LDS operations of chunk kc (clamped past the end: the count per chunk is fixed)
  auto issue_x = [&](int kc, int slot) {
    const uint32_t koff = (uint32_t)min(kc, KC - 1) * 128u;
    const u32x4 xo = *(const u32x4*)xoff_lds[tid];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      dma16_global_to_lds(p.a, xo[i] + koff, x_dst0 + slot * kXSlot + i * 1024);
    if constexpr (QT == 0) {
      dma4_global_to_lds_masked<0xffffffffull>(p.a_scale, sc_voff + (uint32_t)min(kc, KC - 1) * 4u,
                                               sc_dst0 + slot * kScSlot);
    }
  };

  // ---- fragment reads of the activations: lane (j, h), row tile rt, pieces 2q + h at
  // physical piece (2q + h) ^ ((j >> 1) & 7): byte offsets f0 ^ (32 q)
  const int f0 = j * 128 + (((h ^ (j >> 1)) & 7) << 4);
  // the two pieces of chunk half hk of row tile rt
  auto read_x = [&](int slot, int rt, int hk, u32x4 (&x)[2]) {
    const unsigned char* base = x_lds + slot * kXSlot + rt * 4096;
    x[0] = *(const u32x4*)(base + (f0 ^ (hk << 6)));
    x[1] = *(const u32x4*)(base + (f0 ^ (hk << 6) ^ 32));
  };
  // max(scale, floor) as ONE integer maximum on the bit patterns (positive floats order like
  // their bits; a negative or zero scale becomes the floor): fmaxf costs a second instruction
  // that quiets NaNs, and these sit in the main loop
  auto floor_scale = [&](float v, float floor_v) -> float {
    return __int_as_float(max(__float_as_int(v), __float_as_int(floor_v)));
  };
  // row 32 rt + j's activation scale sits in wave rt's strip of the chunk's slot
  const unsigned char* as_mine = sc_lds + j * 4;
  auto read_as = [&](int slot, int rt) -> float {
    return floor_scale(*(const float*)(as_mine + slot * kScSlot + rt * kScWave), kActScaleFloor);
  };
  // (wave-uniform)
  auto read_ws = [&](int kc, int ct) -> float {
    return floor_scale(ws_lds[wave][ct][kc], kWScaleFloor);
  };

  f32x16 acc[NRT][2];  // [row tile][column tile]
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][ct][r] = 0.0f;

  // both MFMAs (fp8: one per column tile; 16 bit: two per column tile) of one (row tile, half)
  auto mma = [&](f32x16& a, const u32x4 (&b)[2], const u32x4 (&x)[2]) {
    if constexpr (QT == 0) {
      a = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cat8(b[0], b[1]), cat8(x[0], x[1]), a, 0, 0,
                                                          0, 0, 0, 0);
    } else {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        if constexpr (DT == DLB_DTYPE_BF16)
          a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[q]),
                                                      __builtin_bit_cast(bf16x8, x[q]), a, 0, 0, 0);
        else
          a = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b[q]),
                                                     __builtin_bit_cast(f16x8, x[q]), a, 0, 0, 0);
      }
    }
  };
  auto scale_tile = [&](f32x16& a, float f) {
#pragma unroll
    for (int r = 0; r < 16; ++r) a[r] *= f;
    // keep the multiplies where they are written (between two MFMAs); the optimiser would
    // otherwise sink them into one long run with nothing to overlap
    asm volatile("" : "+v"(a));
  };

  // Order of the vector-memory operations of a wave, per chunk k (the prologue plays the first
  // two chunks):   W(k, half 0) [4]   X(k) [D]   W(k, half 1) [4]
  // Operations complete in order, so "at most n outstanding" means everything but the youngest
  // n has landed.
  issue_x(0, 0);
  issue_w(H1{}, 0, wr[0][1]);
  issue_w(H0{}, 1, wr[1][0]);
  issue_x(1, 1);
  issue_w(H1{}, 1, wr[1][1]);
  wait_vm<12 + D>();  // X(0) landed
  __syncthreads();

  u32x4 xa[2], xb[2];  // fragment buffers: row tiles 0 and 2 use xa, 1 and 3 use xb
  read_x(0, 0, 0, xa);
  // s(k) / s(k + 1), k and k + 1 being the chunks in slots `cur` and `nxt` (both chunks' scales
  // are in LDS), split by operand: the activation part of row tile rt is computed where it is
  // used, so that it does not stay in a register across the chunk; the block-scale part of
  // column tile ct is wave-uniform and lives in a scalar register
  auto ratio_a = [&](int cur, int nxt, int rt) -> float {
    return read_as(cur, rt) * __builtin_amdgcn_rcpf(read_as(nxt, rt));
  };
  // (kept as bit patterns: integers that come out of readfirstlane stay in scalar registers)
  auto ratio_w = [&](int kc, int ct) -> unsigned int {  // chunk kc -> kc + 1
    const float r = read_ws(kc, ct) * __builtin_amdgcn_rcpf(read_ws(kc + 1, ct));
    return (unsigned int)__builtin_amdgcn_readfirstlane(__float_as_uint(r));
  };
  unsigned int rw_in[2] = {0x3f800000u, 0x3f800000u};   // chunk k - 1 -> k (used in chunk k's first half)
  unsigned int rw_out[2] = {0x3f800000u, 0x3f800000u};  // chunk k -> k + 1 (used in its second half)

  int x_cur = 0, x_nxt = 1, x_tgt = 2;  // slots of chunks k, k + 1, k + 2

  // Chunk k.  On entry xa = X(k, row tile 0, half 0).  The multiplies that move an accumulator
  // tile from the scale of chunk k to that of chunk k + 1 sit behind the MFMAs of the following
  // row tile in the chunk's second half (the tile's own MFMA has finished by then), those of the
  // last row tile behind the first MFMAs of chunk k + 1.
  auto chunk = [&](auto ptag, int k) {
    constexpr int P = decltype(ptag)::value;
    const bool first = k == 0, more = k + 1 < KC;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      // even row tiles compute from xa, odd ones from xb; the next step's fragments are fetched
      // into the other buffer before this step's MFMAs ((row tile 0, half 1) after the last)
      u32x4(&xc)[2] = (rt & 1) ? xb : xa;
      u32x4(&xn)[2] = (rt & 1) ? xa : xb;
      if (rt + 1 < NRT) read_x(x_cur, rt + 1, 0, xn);
      else read_x(x_cur, 0, 1, xn);
      __builtin_amdgcn_sched_barrier(0);
      // (the previous chunk's scales sit in the slot that is refilled after this chunk's barrier)
      float al = 1.0f;
      if (QT == 0 && rt == 0 && !first) al = ratio_a(x_tgt, x_cur, NRT - 1);
      mma(acc[rt][0], wr[P][0][0], xc);
      if (QT == 0 && rt == 0 && !first) scale_tile(acc[NRT - 1][0], al * __uint_as_float(rw_in[0]));
      mma(acc[rt][1], wr[P][0][1], xc);
      if (QT == 0 && rt == 0 && !first) scale_tile(acc[NRT - 1][1], al * __uint_as_float(rw_in[1]));
      __builtin_amdgcn_sched_barrier(0);
    }
    issue_w(H0{}, k + 2, wr[P][0]);
    wait_vm<8>();     // this wave's part of X(k + 1) landed
    __syncthreads();  // X(k + 1) complete; every wave is done reading X(k - 1)
    if (QT == 0 && more) {
      rw_out[0] = ratio_w(k, 0);
      rw_out[1] = ratio_w(k, 1);
    }
    issue_x(k + 2, x_tgt);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      u32x4(&xc)[2] = (rt & 1) ? xb : xa;
      u32x4(&xn)[2] = (rt & 1) ? xa : xb;
      if (rt + 1 < NRT) read_x(x_cur, rt + 1, 1, xn);
      else if (more) read_x(x_nxt, 0, 0, xn);
      __builtin_amdgcn_sched_barrier(0);
      float ap = 1.0f;
      if (QT == 0 && rt > 0 && more) ap = ratio_a(x_cur, x_nxt, rt - 1);
      mma(acc[rt][0], wr[P][1][0], xc);
      if (QT == 0 && rt > 0 && more) scale_tile(acc[rt - 1][0], ap * __uint_as_float(rw_out[0]));
      mma(acc[rt][1], wr[P][1][1], xc);
      if (QT == 0 && rt > 0 && more) scale_tile(acc[rt - 1][1], ap * __uint_as_float(rw_out[1]));
      __builtin_amdgcn_sched_barrier(0);
    }
    issue_w(H1{}, k + 2, wr[P][1]);
    rw_in[0] = rw_out[0];
    rw_in[1] = rw_out[1];
    const int xr = x_cur;
    x_cur = x_nxt;
    x_nxt = x_tgt;
    x_tgt = xr;
  };
  // two chunks per iteration, so that every weight unit has a fixed home in the register file
  // The wave runs its main loop at a raised priority: when the CU's other workgroup is in its
  // prologue or epilogue (vector arithmetic, no matrix work), this wave's MFMAs win the issue slot
  // they share (gate_up 2 - 3 % faster, down unchanged).
  __builtin_amdgcn_s_setprio(3);
  int k = 0;
#pragma nounroll
  for (; k + 1 < KC; k += 2) {
    chunk(std::integral_constant<int, 0>{}, k);
    chunk(std::integral_constant<int, 1>{}, k + 1);
  }
  if (k < KC) chunk(std::integral_constant<int, 0>{}, k);
  __builtin_amdgcn_s_setprio(0);
  // the clamped copies past the end are still in flight and will write the LDS slots
  wait_vm<0>();
  // the accumulators hold sum / s(last chunk), whose scales are still in their LDS slot (x_tgt
  // after the last rotation): final scale of tile (rt, ct)
  auto final_scale = [&](int rt, int ct) -> float {
    return QT == 0 ? read_as(x_tgt, rt) * read_ws(KC - 1, ct) : 1.0f;
  };

  // The lane coordinates are derived afresh for the epilogue: carried across the main loop they
  // would hold four registers that the loop needs.
  int tid_e = threadIdx.x;
  asm volatile("" : "+v"(tid_e));
  const int j_e = tid_e & 31, h_e = (tid_e >> 5) & 1;
  // ---- epilogues: lane holds token (32*rt + j_e), columns ncol[ct] + 8*(r/4) + 4*h_e + r%4.
  // A swap between the lane halves turns two 4-column runs into one 8-column run per lane.
  // Output tiles leave through LDS (the activation slots, free once every wave has left the
  // main loop and drained its copies) as whole rows, adjacent lanes on adjacent 16-byte pieces.
  if (GATED && QT == 1) {
    // rounding points of the reference pipeline (fused_moe.py:166,351-352): GEMM result,
    // silu(gate) and the product are each rounded to the activation type
    constexpr int kActPitch = 256 + 16;
    static_assert(128 * kActPitch <= NX * kXSlot, "output staging fits the activation slots");
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      {
        unsigned short* dst = (unsigned short*)(x_lds + (32 * rt + j_e) * kActPitch) + wave * 32 + 8 * h_e;
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
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // 128 rows x 16 pieces of 16 bytes
      const int r = (tid_e >> 4) + 16 * i, pc = tid_e & 15;
      if (r < 32 * NRT && nt * 128 + 8 * pc < p.I)  // (the last column tile may be partial)
        *(u32x4*)((unsigned short*)p.hq + (int64_t)(row0 + r) * p.I + nt * 128 + 8 * pc) =
            *(const u32x4*)(x_lds + r * kActPitch + 16 * pc);
    }
  } else if (GATED) {
    constexpr int kGatedPitch = 128 + 16;  // staging row pitch of the fp8 output tile
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      {
        const float sg = final_scale(rt, 0), su = final_scale(rt, 1);
        float amax = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float gate = acc[rt][0][r] * sg;
          const float up = acc[rt][1][r] * su;
          const float v = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;  // 1-ulp reciprocal
          acc[rt][0][r] = v;
          amax = fmaxf(amax, fabsf(v));
        }
        amax = max_xor32(amax);
        if (h_e == 0) red_lds[wave][32 * rt + j_e] = amax;
      }
    }
    __syncthreads();  // row maxima visible; every wave has left the main loop
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      {
        const int r = 32 * rt + j_e;
        const float m = fmaxf(fmaxf(red_lds[0][r], red_lds[1][r]), fmaxf(red_lds[2][r], red_lds[3][r]));
        const float scale = fmaxf(m, kQuantEps) / kFp8Max;
        const float inv = __builtin_amdgcn_rcpf(scale);  // the stored scale stays exact
        unsigned int q[4];
#pragma unroll
        for (int s = 0; s < 4; ++s)
          q[s] = pack4_fp8(acc[rt][0][4 * s] * inv, acc[rt][0][4 * s + 1] * inv,
                           acc[rt][0][4 * s + 2] * inv, acc[rt][0][4 * s + 3] * inv);
        swap_halves(q[0], q[1]);
        swap_halves(q[2], q[3]);
        unsigned char* dst = x_lds + r * kGatedPitch + wave * 32 + 8 * h_e;
        *(u32x2*)(dst) = u32x2{q[0], q[1]};
        *(u32x2*)(dst + 16) = u32x2{q[2], q[3]};
        if (wave == 0 && h_e == 0) p.hs[(int64_t)(row0 + r) * (p.I >> 7) + nt] = scale;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // 128 rows x 8 pieces of 16 bytes
      const int r = (tid_e >> 3) + 32 * i, pc = tid_e & 7;
      if (r < 32 * NRT)
        *(u32x4*)(p.hq + (int64_t)(row0 + r) * p.I + nt * 128 + 16 * pc) =
            *(const u32x4*)(x_lds + r * kGatedPitch + 16 * pc);
    }
  } else {
    // the 128 x 256 output tile goes out 64 rows at a time
    constexpr int kPitch = 512 + 16;  // staging row pitch: rows 16 bytes apart in the banks
    static_assert(64 * kPitch <= NX * kXSlot, "output staging fits the activation slots");
    const int ncols = min(256, p.N - nt * 256);
    __syncthreads();  // every wave has left the main loop
#pragma unroll
    for (int half = 0; half < NRT / 2; ++half) {
      {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          const int rt = 2 * half + rr;
          {
            const float rwt = rw_lds[32 * rt + j_e];
#pragma unroll
            for (int ct = 0; ct < 2; ++ct) {
              const float f = rwt * final_scale(rt, ct);
#pragma unroll
              for (int pr = 0; pr < 2; ++pr) {
                unsigned int o[2][2];
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                  const int r = 4 * (2 * pr + s);
                  o[s][0] = Elem<DT>::pack(acc[rt][ct][r] * f, acc[rt][ct][r + 1] * f);
                  o[s][1] = Elem<DT>::pack(acc[rt][ct][r + 2] * f, acc[rt][ct][r + 3] * f);
                }
                swap_halves(o[0][0], o[1][0]);
                swap_halves(o[0][1], o[1][1]);
                *(u32x4*)(x_lds + (32 * rr + j_e) * kPitch + (wave * 64 + ct * 32 + 16 * pr + 8 * h_e) * 2) =
                    u32x4{o[0][0], o[0][1], o[1][0], o[1][1]};
              }
            }
          }
        }
        __syncthreads();
        // 64 rows x 32 pieces; thread t takes piece t % 32 of rows t / 32 + 8 i
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int r = (tid_e >> 5) + 8 * i, pc = tid_e & 31;
          const int sid = sid_lds[64 * half + r];  // destination row
          if (sid >= 0 && 8 * pc < ncols)
            // (non-temporal: the 100 MB of slot rows would otherwise push the weight lines that the
            // expert's other row blocks are about to read out of L2)
            __builtin_nontemporal_store(
                *(const u32x4*)(x_lds + r * kPitch + 16 * pc),
                (u32x4*)((unsigned short*)p.out + (int64_t)sid * p.N + nt * 256 + 8 * pc));
        }
        if (half + 1 < NRT / 2) __syncthreads();  // the second half reuses the staging rows
      }
    }
  }
  };  // run
  if (tile.rows > 64) run(std::integral_constant<int, 4>{});
  else run(std::integral_constant<int, 2>{});
}

// out[t, n] = sum_j in[t * topk + j, n], fp32 accumulation in slot order, one rounding.
// TOPK > 0: the slot count is a compile-time constant and all its loads are requested before the
// first is used (the kernel is a pure stream: what counts is the number of bytes in flight);
// TOPK = 0: any slot count, four loads at a time.
template <int DT, int TOPK>
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
  auto add = [&](const u32x4& v) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      s[2 * w] += Elem<DT>::lo(v[w]);
      s[2 * w + 1] += Elem<DT>::hi(v[w]);
    }
  };
  const u32x4* row = in + t * (int64_t)(TOPK ? TOPK : topk) * vec_per_row + col;
  if constexpr (TOPK > 0) {
    u32x4 v[TOPK];
#pragma unroll
    for (int j = 0; j < TOPK; ++j) v[j] = __builtin_nontemporal_load(row + (int64_t)j * vec_per_row);
#pragma unroll
    for (int j = 0; j < TOPK; ++j) add(v[j]);
  } else {
    int j = 0;
    for (; j + 4 <= topk; j += 4) {
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(row + (int64_t)(j + u) * vec_per_row);
#pragma unroll
      for (int u = 0; u < 4; ++u) add(v[u]);
    }
    for (; j < topk; ++j) add(__builtin_nontemporal_load(row + (int64_t)j * vec_per_row));
  }
  u32x4 r;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = Elem<DT>::pack(s[2 * w], s[2 * w + 1]);
  __builtin_nontemporal_store(r, out + i);
}

}  // namespace
}  // namespace dlb


extern "C" int dlb_per_token_group_quant_fp8(const void* x, void* xq, float* xs, int64_t M,
                                             int K, int64_t ld_x, int64_t ld_q, int64_t ld_s,
                                             int dtype, void* stream) {
  using namespace dlb;
  QuantParams q;
  const int st = fill_quant_params(q, x, xq, xs, M, K, ld_x, ld_q, ld_s, dtype);
  if (st != DLB_OK) return st;
  if (M == 0 || K == 0) return DLB_OK;
  const dim3 grid((uint32_t)ceil_div(q.total_groups, kQuantGroupsPerBlock));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DLB_DTYPE_BF16)
    hipLaunchKernelGGL(quant_fp8_group128_kernel<DLB_DTYPE_BF16>, grid, dim3(kQuantThreads), 0, s, q);
  else
    hipLaunchKernelGGL(quant_fp8_group128_kernel<DLB_DTYPE_F16>, grid, dim3(kQuantThreads), 0, s, q);
  return launch_status();
}

namespace dlb {
namespace {

template <bool GATED, int QT>
int launch_moe_gemm(const MoeGemmParams& p, int dtype, int w_layout, hipStream_t s) {
  // one workgroup per tile slot of the block capacity; a workgroup finds its tile from the
  // expert counts (or finds none and leaves), in the order described at find_tile
  if (w_layout && p.N % 16 != 0) return DLB_ERR_UNSUPPORTED;  // operand order comes in 16-row tiles
  const uint32_t grid = (uint32_t)(ceil_div((int64_t)p.num_mblocks * p.num_ntiles, 8) * 8);
#define DLB_LAUNCH_GEMM(DT_)                                                                   \
  do {                                                                                       \
    if (w_layout)                                                                            \
      hipLaunchKernelGGL((moe_gemm_kernel<GATED, DT_, QT, 1>), dim3(grid), dim3(256), 0, s, p); \
    else                                                                                     \
      hipLaunchKernelGGL((moe_gemm_kernel<GATED, DT_, QT, 0>), dim3(grid), dim3(256), 0, s, p); \
  } while (0)
  if (dtype == DLB_DTYPE_BF16) DLB_LAUNCH_GEMM(DLB_DTYPE_BF16);
  else if (dtype == DLB_DTYPE_F16) DLB_LAUNCH_GEMM(DLB_DTYPE_F16);
  else return DLB_ERR_UNSUPPORTED;
#undef DLB_LAUNCH_GEMM
  return launch_status();
}

// shared argument checks and parameter block of the four grouped-GEMM entry points;
// elem = bytes per operand element (1 for fp8, 2 for bf16/f16); N_out = weight rows per expert
// of the down GEMM (the output width)
int fill_gemm_params(MoeGemmParams& p, bool gated, int elem, const void* a, const float* a_scale,
                     const void* w, const float* w_scale, const int32_t* sorted_ids,
                     const int32_t* expert_counts, int num_experts, int num_mblocks, int block_m,
                     int num_tokens, int topk, int H, int I, int expert_offset,
                     int num_local_experts) {
  const int Kel = gated ? H : I;       // reduction length (elements)
  const int N = gated ? 2 * I : H;     // weight rows per expert
  if (num_mblocks < 0 || H < 1 || I < 1) return DLB_ERR_BAD_ARG;
  if (num_mblocks == 0) return DLB_OK;
  if (!a || !w || !sorted_ids || !expert_counts) return DLB_ERR_BAD_ARG;
  if (elem == 1 && (!a_scale || !w_scale)) return DLB_ERR_BAD_ARG;
  if (num_tokens < 1 || topk < 1 || num_local_experts < 1 || num_experts < 1) return DLB_ERR_BAD_ARG;
  if (expert_offset < 0 || expert_offset + num_local_experts > num_experts) return DLB_ERR_BAD_ARG;
  if (num_experts > 256) return DLB_ERR_UNSUPPORTED;  // four experts per lane in the tile look-up
  if (block_m != 64 && block_m != 128) return DLB_ERR_UNSUPPORTED;
  // a row must be a whole number of 128-byte chunks.  fp8: the scale groups and the re-quantised
  // column tiles are 128 wide; 16 bit: a partial last column tile is masked, so 64-element
  // multiples do (both reduction lengths) and the output width only has to fill 16-byte stores
  if (elem == 1 ? (H % 128 != 0 || I % 128 != 0) : (Kel % 64 != 0 || I % 64 != 0 || H % 8 != 0))
    return DLB_ERR_UNSUPPORTED;
  // fp8: the block scales of all K chunks of a tile are parked in LDS
  if (elem == 1 && Kel / 128 > kMoeMaxKChunks) return DLB_ERR_UNSUPPORTED;
  if (!aligned16(a) || !aligned16(w)) return DLB_ERR_UNSUPPORTED;
  if ((int64_t)N * Kel * elem >= (int64_t)0xffffffffu) return DLB_ERR_UNSUPPORTED;  // 32-bit lane offsets
  const int64_t a_rows = gated ? num_tokens : (int64_t)num_mblocks * block_m;
  if (a_rows * Kel * elem >= (int64_t)0xffffffffu) return DLB_ERR_UNSUPPORTED;
  if ((int64_t)num_mblocks * block_m >= (int64_t)0x7fffffff ||
      (int64_t)num_tokens * topk >= (int64_t)0x7fffffff)
    return DLB_ERR_UNSUPPORTED;
  p = MoeGemmParams{};
  p.a = (const unsigned char*)a;
  p.a_scale = a_scale;
  p.w = (const unsigned char*)w;
  p.w_scale = w_scale;
  p.sorted_ids = IdxArray{sorted_ids, 0};
  p.counts = IdxArray{expert_counts, 0};
  p.seg_start = IdxArray{nullptr, 0};
  p.a_rows = a_rows;
  p.gather_a = 0;   // (the gated kernel always gathers; the down GEMMs read sorted rows)
  p.scatter_c = 1;
  p.num_experts = num_experts;
  p.num_mblocks = num_mblocks;
  p.bm_shift = block_m == 128 ? 7 : 6;
  p.num_ntiles = gated ? (int)ceil_div(I, 128) : (int)ceil_div(H, 256);
  p.K = Kel * elem;
  p.N = N;
  p.KC = p.K / 128;
  p.topk = topk;
  p.numel = num_tokens * topk;
  p.num_tokens = num_tokens;
  p.expert_offset = expert_offset;
  p.num_local = num_local_experts;
  p.I = I;
  return DLB_OK;
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_moe_gemm_fp8_gate_up(const void* xq, const float* xs, const void* w1q,
                                        const float* w1s, const int32_t* sorted_ids,
                                        const int32_t* expert_counts, int num_experts,
                                        int num_mblocks, int block_m, int num_tokens, int topk,
                                        int H, int I, int expert_offset, int num_local_experts,
                                        int w_layout, void* hq, float* hs, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, true, 1, xq, xs, w1q, w1s, sorted_ids, expert_counts,
                                  num_experts, num_mblocks, block_m, num_tokens, topk, H, I,
                                  expert_offset, num_local_experts);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!hq || !hs) return DLB_ERR_BAD_ARG;
  if (!aligned16(hq)) return DLB_ERR_UNSUPPORTED;
  p.hq = (unsigned char*)hq;
  p.hs = hs;
  return launch_moe_gemm<true, 0>(p, DLB_DTYPE_BF16, w_layout, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_fp8_down(const void* hq, const float* hs, const void* w2q,
                                     const float* w2s, const int32_t* sorted_ids,
                                     const int32_t* expert_counts, int num_experts,
                                     const float* topk_weights, int num_mblocks, int block_m,
                                     int num_tokens, int topk, int H, int I, int expert_offset,
                                     int num_local_experts, int w_layout, void* out,
                                     int out_dtype, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, false, 1, hq, hs, w2q, w2s, sorted_ids, expert_counts,
                                  num_experts, num_mblocks, block_m, num_tokens, topk, H, I,
                                  expert_offset, num_local_experts);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!out || !topk_weights) return DLB_ERR_BAD_ARG;
  if (!aligned16(out)) return DLB_ERR_UNSUPPORTED;
  p.out = out;
  p.topk_w = topk_weights;
  return launch_moe_gemm<false, 0>(p, out_dtype, w_layout, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_16bit_gate_up(const void* x, const void* w1,
                                          const int32_t* sorted_ids, const int32_t* expert_counts,
                                          int num_experts, int num_mblocks, int block_m,
                                          int num_tokens, int topk, int H, int I,
                                          int expert_offset, int num_local_experts, int w_layout,
                                          void* act, int dtype, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, true, 2, x, nullptr, w1, nullptr, sorted_ids, expert_counts,
                                  num_experts, num_mblocks, block_m, num_tokens, topk, H, I,
                                  expert_offset, num_local_experts);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!act) return DLB_ERR_BAD_ARG;
  if (!aligned16(act)) return DLB_ERR_UNSUPPORTED;
  p.hq = (unsigned char*)act;
  return launch_moe_gemm<true, 1>(p, dtype, w_layout, (hipStream_t)stream);
}

extern "C" int dlb_moe_gemm_16bit_down(const void* act, const void* w2,
                                       const int32_t* sorted_ids, const int32_t* expert_counts,
                                       int num_experts, const float* topk_weights,
                                       int num_mblocks, int block_m, int num_tokens, int topk,
                                       int H, int I, int expert_offset, int num_local_experts,
                                       int w_layout, void* out, int dtype, void* stream) {
  using namespace dlb;
  MoeGemmParams p;
  const int st = fill_gemm_params(p, false, 2, act, nullptr, w2, nullptr, sorted_ids,
                                  expert_counts, num_experts, num_mblocks, block_m, num_tokens,
                                  topk, H, I, expert_offset, num_local_experts);
  if (st != DLB_OK || num_mblocks == 0) return st;
  if (!out || !topk_weights) return DLB_ERR_BAD_ARG;
  if (!aligned16(out)) return DLB_ERR_UNSUPPORTED;
  p.out = out;
  p.topk_w = topk_weights;
  return launch_moe_gemm<false, 1>(p, dtype, w_layout, (hipStream_t)stream);
}

// The reference's grouped-GEMM launcher in its own argument form (16-bit operands):
// C[row] = A[row'] . B[e]^T (x weights[slot]) for every routing slot of the expert-sorted list.
extern "C" int dlb_moe_gemm_16bit_launcher(const void* a, const void* b, void* c,
                                           const void* sorted_idx, const void* exp_start,
                                           const void* exp_end, int index64_mask,
                                           const float* weights, int num_experts,
                                           int expert_offset, int num_local_experts,
                                           int64_t num_slots, int64_t a_rows, int topk, int N,
                                           int K, int reindex_a, int reindex_c, int dtype,
                                           void* stream) {
  using namespace dlb;
  if (num_slots < 0 || a_rows < 0 || topk < 1 || N < 1 || K < 1) return DLB_ERR_BAD_ARG;
  if (num_experts < 1 || num_local_experts < 1 || expert_offset < 0 ||
      expert_offset + num_local_experts > num_experts)
    return DLB_ERR_BAD_ARG;
  if (index64_mask & ~7) return DLB_ERR_BAD_ARG;
  if (num_slots == 0) return DLB_OK;
  if (!a || !b || !c || !sorted_idx || !exp_start || !exp_end || a_rows < 1) return DLB_ERR_BAD_ARG;
  if (num_experts > 256) return DLB_ERR_UNSUPPORTED;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
  // rows are whole 128-byte chunks (64 elements); outputs leave in 16-byte pieces
  if (K % 64 != 0 || N % 8 != 0) return DLB_ERR_UNSUPPORTED;
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return DLB_ERR_UNSUPPORTED;
  if ((int64_t)N * K * 2 >= (int64_t)0xffffffffu || a_rows * K * 2 >= (int64_t)0xffffffffu ||
      num_slots >= (int64_t)0x7fffffff)
    return DLB_ERR_UNSUPPORTED;
  MoeGemmParams p = MoeGemmParams{};
  p.a = (const unsigned char*)a;
  p.w = (const unsigned char*)b;
  p.sorted_ids = idx_array(sorted_idx, index64_mask, 0);
  p.seg_start = idx_array(exp_start, index64_mask, 1);
  p.counts = idx_array(exp_end, index64_mask, 2);   // segment ends: find_tile subtracts the starts
  p.num_experts = num_experts;
  p.bm_shift = 7;
  // every expert's segment is cut into blocks of 128 rows of its own: at most one partial block each
  p.num_mblocks = (int)(ceil_div(num_slots, 128) + num_local_experts);
  p.num_ntiles = (int)ceil_div(N, 256);
  p.K = K * 2;
  p.N = N;
  p.KC = p.K / 128;
  p.topk = topk;
  p.numel = (int)num_slots;
  // gathered rows are slot / topk; the caller says how many rows `a` has
  p.num_tokens = a_rows < 0x7fffffff ? (int)a_rows : 0x7fffffff;
  p.a_rows = a_rows;
  p.expert_offset = expert_offset;
  p.num_local = num_local_experts;
  p.I = 0;
  p.gather_a = reindex_a ? 1 : 0;
  p.scatter_c = reindex_c ? 1 : 0;
  p.out = c;
  p.topk_w = weights;  // null: no routing weights
  return launch_moe_gemm<false, 1>(p, dtype, 0, (hipStream_t)stream);
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
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16) return DLB_ERR_UNSUPPORTED;
#define DLB_LAUNCH_SUM(DT_, TK_)                                                                  \
  hipLaunchKernelGGL((moe_topk_sum_kernel<DT_, TK_>), grid, dim3(256), 0, s, (const u32x4*)in, \
                     (u32x4*)out, total, (int)(N / 8), topk)
#define DLB_DISPATCH_SUM(DT_)                 \
  switch (topk) {                             \
    case 1: DLB_LAUNCH_SUM(DT_, 1); break;    \
    case 2: DLB_LAUNCH_SUM(DT_, 2); break;    \
    case 4: DLB_LAUNCH_SUM(DT_, 4); break;    \
    case 6: DLB_LAUNCH_SUM(DT_, 6); break;    \
    case 8: DLB_LAUNCH_SUM(DT_, 8); break;    \
    default: DLB_LAUNCH_SUM(DT_, 0); break;   \
  }
  if (dtype == DLB_DTYPE_BF16) { DLB_DISPATCH_SUM(DLB_DTYPE_BF16) } else { DLB_DISPATCH_SUM(DLB_DTYPE_F16) }
#undef DLB_DISPATCH_SUM
#undef DLB_LAUNCH_SUM
  return launch_status();
}
