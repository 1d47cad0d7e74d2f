// Expert alignment of MoE routing for gfx950: per-expert counts, expert-sorted flat slot ids
// padded per expert to a multiple of `block`, and the expert id of each block.
//
// The reference derives the same information with a full argsort of the flat id list plus a
// kernel that rescans that list once per expert
// (python/dlBLAS/dlblas/kernels/fused_moe.py:238-293, 314-320: exp_start/exp_end are the
// exclusive/inclusive cumulative sums of the per-expert counts).  Here it is a counting sort:
//   1. count:  every workgroup histograms its contiguous chunk of the flat id list in LDS and
//              writes one row of per-chunk counts (plain stores, so the result is reproducible);
//   2. scan:   one workgroup turns the [chunks, E] table into per-chunk start offsets, pads each
//              expert's total to `block`, and emits counts, block -> expert ids, the sentinel
//              pad slots and the padded total;
//      (for up to 256 chunks step 2 is folded into step 3: every workgroup reduces the small
//      count table itself, which saves a launch on the sizes a decoder layer produces)
//   3. place:  every workgroup re-reads its chunk in order and writes flat index i to
//              start[chunk][e] + (number of earlier i' in the chunk with the same e), the rank
//              coming from wave ballots, which makes the sort stable (ascending i per expert).
// Integer work only; no float or order-dependent atomics, so the output is bit-reproducible.
#include <mutex>

#include "common.h"
#include "quant_fp8.h"

namespace dlb {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kChunk = 2048;  // flat ids per workgroup (large inputs)
constexpr int kMaxE = 256;
constexpr int kFusedChunks = 256;  // rows of the count table the fused placement kernel reduces
static_assert(kFusedChunks == kRouteMaxChunks, "the fused router sizes its chunks for this table");

// Flat ids per chunk (= per workgroup of the counting and the placement pass).  Inputs of up to
// kFusedChunks * kChunk ids are cut into as many chunks as the fused placement kernel takes (256),
// but not below one tile of 256 ids: a decoder layer's 25 k - 100 k routing slots then run on
// 96 - 256 workgroups with one or two tiles each instead of 12 - 48 workgroups that walk eight
// tiles one after the other.  Larger inputs use chunks of kChunk ids and the three-launch path.
__host__ __device__ inline int chunk_ids_for(int64_t numel) {
  if (numel > (int64_t)kFusedChunks * kChunk) return kChunk;
  const int64_t per = (numel + kFusedChunks - 1) / kFusedChunks;
  const int64_t rounded = (per + 63) / 64 * 64;
  return (int)(rounded < kThreads ? kThreads : rounded);
}
__host__ __device__ inline int64_t num_chunks(int64_t numel) {
  const int c = chunk_ids_for(numel);
  return numel > 0 ? (numel + c - 1) / c : 1;
}

__global__ __launch_bounds__(kThreads) void align_count_kernel(const IdxArray ids,
                                                               int64_t numel, int E, int chunk_ids,
                                                               int32_t* __restrict__ chunk_counts) {
  __shared__ int32_t hist[kMaxE];
  for (int e = threadIdx.x; e < E; e += kThreads) hist[e] = 0;
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * chunk_ids;
  const int64_t end = begin + chunk_ids < numel ? begin + chunk_ids : numel;
  for (int64_t i = begin + threadIdx.x; i < end; i += kThreads) {
    const int32_t e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&hist[e], 1);  // integer add: order-insensitive
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kThreads) chunk_counts[(int64_t)blockIdx.x * E + e] = hist[e];
}

// One workgroup of 1024 threads: sub-group q = tid / E' (E' = E rounded up to 64) scans a
// slice of the chunk rows for expert tid % E', the slices are combined through LDS, so the
// dependent chain per thread is chunks / groups long instead of chunks.
constexpr int kScanThreads = 1024;

__global__ __launch_bounds__(kScanThreads) void align_scan_kernel(
    int32_t* __restrict__ chunk_counts /* in: counts, out: start offsets */, int64_t chunks, int E,
    int block, int32_t numel, int32_t* __restrict__ sorted_ids, int64_t sorted_cap,
    int32_t* __restrict__ expert_ids, int64_t expert_ids_cap, int32_t* __restrict__ counts,
    int32_t* __restrict__ num_post_pad) {
  __shared__ int32_t part_s[kScanThreads];  // [group][expert'] slice totals -> slice bases
  __shared__ int32_t total_s[kMaxE];
  __shared__ int32_t base_s[kMaxE + 1];
  const int tid = threadIdx.x;
  const int ep = (E + 63) & ~63;           // experts rounded up to a whole wave
  const int groups = kScanThreads / ep;     // >= 4 for E <= 256
  const int e = tid % ep, q = tid / ep;
  const bool live = (e < E) && (q < groups);
  const int64_t per = (chunks + groups - 1) / groups;
  const int64_t c0 = q * per, c1 = (c0 + per < chunks) ? c0 + per : chunks;

  int32_t slice = 0;
  if (live)
    for (int64_t c = c0; c < c1; ++c) slice += chunk_counts[c * E + e];
  part_s[tid] = slice;
  __syncthreads();
  if (tid < E) {  // exclusive scan over the groups of this expert, total
    int32_t run = 0;
    for (int g2 = 0; g2 < groups; ++g2) {
      const int32_t v = part_s[g2 * ep + tid];
      part_s[g2 * ep + tid] = run;
      run += v;
    }
    total_s[tid] = run;
  }
  __syncthreads();
  if (tid < 64) {  // padded totals -> expert bases: wave scan over up to 256 experts
    int32_t run = 0;
    for (int i0 = 0; i0 < E; i0 += 64) {
      const int i = i0 + tid;
      const int32_t padded = (i < E) ? (int32_t)(ceil_div(total_s[i], block) * block) : 0;
      int32_t incl = padded;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int32_t up = __shfl_up(incl, d);
        if (tid >= d) incl += up;
      }
      if (i < E) base_s[i] = run + incl - padded;
      run += __shfl(incl, 63);
    }
    if (tid == 0) {
      base_s[E] = run;
      *num_post_pad = run;
    }
  }
  __syncthreads();
  const int32_t total_padded = base_s[E];
  if (live) {
    // chunk start offsets of this slice for the placement pass
    int32_t run = base_s[e] + part_s[q * ep + e];
    for (int64_t c = c0; c < c1; ++c) {
      const int32_t n = chunk_counts[c * E + e];
      chunk_counts[c * E + e] = run;
      run += n;
    }
  }
  if (tid < E) {
    const int32_t base = base_s[tid], total = total_s[tid], next = base_s[tid + 1];
    if (counts) counts[tid] = total;
    for (int32_t p = base + total; p < next; ++p) sorted_ids[p] = numel;   // pad slots
    for (int32_t b = base / block; b < next / block; ++b) expert_ids[b] = tid;
  }
  // tails beyond the padded total
  for (int64_t p = (int64_t)total_padded + tid; p < sorted_cap; p += kScanThreads) sorted_ids[p] = numel;
  for (int64_t b = (int64_t)total_padded / block + tid; b < expert_ids_cap; b += kScanThreads)
    expert_ids[b] = -1;
}

__global__ __launch_bounds__(kThreads) void align_place_kernel(
    const IdxArray ids, int64_t numel, int E,
    const int32_t* __restrict__ chunk_start, int32_t* __restrict__ sorted_ids) {
  __shared__ int32_t cursor[kMaxE];           // next free slot per expert for this chunk
  __shared__ int32_t wave_cnt[kWaves][kMaxE];  // per-tile, per-wave counts
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  for (int e = threadIdx.x; e < E; e += kThreads) cursor[e] = chunk_start[(int64_t)blockIdx.x * E + e];
  for (int i = threadIdx.x; i < kWaves * kMaxE; i += kThreads) (&wave_cnt[0][0])[i] = 0;
  __syncthreads();

  const int64_t begin = (int64_t)blockIdx.x * kChunk;
  const int64_t end = begin + kChunk < numel ? begin + kChunk : numel;
  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t tile = begin; tile < end; tile += kThreads) {  // uniform trip count
    const int64_t i = tile + threadIdx.x;
    int32_t e = -1;
    if (i < end) {
      e = ids[i];
      if (e < 0 || e >= E) e = -1;
    }
    // lanes of this wave holding the same expert: intersect ballots over the 9 key bits
    // (bit 8 separates the dropped entries, e = -1 -> key 0x1ff).
    const uint32_t key = (uint32_t)e & 0x1ffu;
    uint64_t peers = ~0ull;
#pragma unroll
    for (int b = 0; b < 9; ++b) {
      const bool bit = (key >> b) & 1u;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const int rank_in_wave = __popcll(peers & lt_mask);
    const int peer_count = __popcll(peers);
    if (e >= 0 && rank_in_wave == 0) wave_cnt[wave][e] = peer_count;
    __syncthreads();
    if (e >= 0) {
      int32_t pos = cursor[e] + rank_in_wave;
      for (int w = 0; w < wave; ++w) pos += wave_cnt[w][e];
      sorted_ids[pos] = (int32_t)i;
    }
    __syncthreads();
    for (int x = threadIdx.x; x < E; x += kThreads) {
      int32_t add = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        add += wave_cnt[w][x];
        wave_cnt[w][x] = 0;
      }
      cursor[x] += add;
    }
    __syncthreads();
  }
}

// Scan and placement in one launch, for inputs of up to kFusedChunks chunks: every workgroup
// reduces the (small) [chunks, E] count table itself -- expert totals, padded expert bases and
// the offsets of its own chunk -- instead of waiting for a separate one-workgroup scan kernel;
// one extra workgroup emits what the scan kernel emits (counts, block -> expert ids, pad slots,
// tails, padded total).  The table is only read here.
struct PlaceParams {
  IdxArray ids;  // int32 or int64 (the routing ids as torch.topk returns them)
  int64_t numel;
  int E, block;
  const int32_t* chunk_counts;
  int chunks, chunk_ids;
  int32_t* sorted_ids;
  int64_t sorted_cap;
  int32_t* expert_ids;
  int64_t expert_ids_cap;
  int32_t* counts;
  int32_t* num_post_pad;
};

// the work of workgroup `me` (0 .. chunks) of the fused scan + placement
__device__ __forceinline__ void align_place_fused_block(const PlaceParams& pp, const int me) {
  const IdxArray ids = pp.ids;
  const int64_t numel = pp.numel;
  const int E = pp.E, block = pp.block, chunks = pp.chunks, chunk_ids = pp.chunk_ids;
  const int32_t* __restrict__ chunk_counts = pp.chunk_counts;
  int32_t* __restrict__ sorted_ids = pp.sorted_ids;
  const int64_t sorted_cap = pp.sorted_cap, expert_ids_cap = pp.expert_ids_cap;
  int32_t* __restrict__ expert_ids = pp.expert_ids;
  int32_t* __restrict__ counts = pp.counts;
  int32_t* __restrict__ num_post_pad = pp.num_post_pad;
  __shared__ int32_t cursor[kMaxE];            // next free slot per expert for this chunk
  __shared__ int32_t wave_cnt[kWaves][kMaxE];  // per-tile, per-wave counts
  __shared__ int32_t total_s[kMaxE];
  __shared__ int32_t base_s[kMaxE + 1];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;

  // this chunk's first ids are requested before the count table is reduced (they do not depend
  // on it), each later tile's while the tile before it is placed
  const int64_t begin = (int64_t)me * chunk_ids;  // chunk_ids flat ids per chunk (kChunk by default)
  const int64_t end = begin + chunk_ids < numel ? begin + chunk_ids : numel;
  auto load_expert = [&](int64_t tile) -> int32_t {
    const int64_t i = tile + tid;
    int32_t e = -1;
    if (i < end) {
      e = ids[i];
      if (e < 0 || e >= E) e = -1;
    }
    return e;
  };
  int32_t e_next = load_expert(begin);

  // totals and the part of them that lies in earlier chunks: sub-group q = tid / E' (E' = E
  // rounded up to a whole wave) sums a slice of the chunk rows for expert tid % E', the slices
  // meet in LDS (wave_cnt doubles as the scratch for that before it is cleared)
  const int ep = (E + 63) & ~63;
  const int groups = kThreads / ep;  // 4, 2 or 1
  {
    const int e = tid % ep, q = tid / ep;
    const int per = (chunks + groups - 1) / groups;
    const int c0 = q * per, c1 = min(c0 + per, chunks);
    int32_t total = 0, before_part = 0;
    if (e < E && q < groups) {
      // The table was written by the launch before this one, on other XCDs: every dependent batch
      // of loads is a full memory round trip.  All rows of the slice are therefore requested at
      // once (64 per thread cover 256 chunks of up to 64 experts; wider expert counts take a
      // second or fourth batch).
      constexpr int kRowsInFlight = 64;
      for (int cb = c0; cb < c1; cb += kRowsInFlight) {
        int32_t n[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u)
          n[u] = (cb + u < c1) ? chunk_counts[(int64_t)(cb + u) * E + e] : 0;
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          total += n[u];
          if (cb + u < me) before_part += n[u];
        }
      }
    }
    int32_t* part = &wave_cnt[0][0];  // [2][groups][ep] <= 2 * 256 entries
    if (q < groups) {
      part[q * ep + e] = total;
      part[kThreads + q * ep + e] = before_part;
    }
  }
  __syncthreads();
  int32_t before = 0;
  if (tid < E) {
    const int32_t* part = &wave_cnt[0][0];
    int32_t total = 0;
    for (int q = 0; q < groups; ++q) {
      total += part[q * ep + tid];
      before += part[kThreads + q * ep + tid];
    }
    total_s[tid] = total;
  }
  __syncthreads();
  for (int i = tid; i < kWaves * kMaxE; i += kThreads) (&wave_cnt[0][0])[i] = 0;
  __syncthreads();
  if (tid < 64) {  // padded totals -> expert bases: wave scan over up to 256 experts
    int32_t run = 0;
    for (int i0 = 0; i0 < E; i0 += 64) {
      const int i = i0 + tid;
      const int32_t padded = (i < E) ? (int32_t)(ceil_div(total_s[i], block) * block) : 0;
      int32_t incl = padded;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int32_t up = __shfl_up(incl, d);
        if (tid >= d) incl += up;
      }
      if (i < E) base_s[i] = run + incl - padded;
      run += __shfl(incl, 63);
    }
    if (tid == 0) base_s[E] = run;
  }
  __syncthreads();
  if (tid < E) cursor[tid] = base_s[tid] + before;
  if (me == chunks) {  // the extra workgroup: what the scan kernel emits besides offsets
    const int32_t total_padded = base_s[E];
    if (tid == 0) *num_post_pad = total_padded;
    if (tid < E) {
      const int32_t base = base_s[tid], total = total_s[tid], next = base_s[tid + 1];
      if (counts) counts[tid] = total;
      for (int32_t q = base + total; q < next; ++q) sorted_ids[q] = (int32_t)numel;  // pad slots
      for (int32_t b = base / block; b < next / block; ++b) expert_ids[b] = tid;
    }
    for (int64_t q = (int64_t)total_padded + tid; q < sorted_cap; q += kThreads)
      sorted_ids[q] = (int32_t)numel;
    for (int64_t b = (int64_t)total_padded / block + tid; b < expert_ids_cap; b += kThreads)
      expert_ids[b] = -1;
    return;
  }
  __syncthreads();

  const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int64_t tile = begin; tile < end; tile += kThreads) {  // uniform trip count
    const int64_t i = tile + tid;
    const int32_t e = e_next;
    e_next = load_expert(tile + kThreads);
    // lanes of this wave holding the same expert: intersect ballots over the 9 key bits
    const uint32_t key = (uint32_t)e & 0x1ffu;
    uint64_t peers = ~0ull;
#pragma unroll
    for (int b = 0; b < 9; ++b) {
      const bool bit = (key >> b) & 1u;
      const uint64_t m = __ballot(bit);
      peers &= bit ? m : ~m;
    }
    const int rank_in_wave = __popcll(peers & lt_mask);
    const int peer_count = __popcll(peers);
    if (e >= 0 && rank_in_wave == 0) wave_cnt[wave][e] = peer_count;
    __syncthreads();
    if (e >= 0) {
      int32_t pos = cursor[e] + rank_in_wave;
      for (int w = 0; w < wave; ++w) pos += wave_cnt[w][e];
      sorted_ids[pos] = (int32_t)i;
    }
    __syncthreads();
    for (int x = tid; x < E; x += kThreads) {
      int32_t add = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        add += wave_cnt[w][x];
        wave_cnt[w][x] = 0;
      }
      cursor[x] += add;
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kThreads) void align_place_fused_kernel(const PlaceParams pp) {
  align_place_fused_block(pp, blockIdx.x);
}

// The fused scan + placement and the fp8 activation quantiser in ONE launch: workgroups
// 0 .. chunks run the placement, the ones after them quantise.  The two jobs share nothing; run
// side by side they cost one launch and the longer of the two instead of two launches.
static_assert(kQuantThreads == kThreads, "one workgroup size for both jobs");
template <int DT>
__global__ __launch_bounds__(kThreads) void align_place_quant_kernel(const PlaceParams pp,
                                                                     const QuantParams q) {
  const int nplace = pp.chunks + 1;
  if ((int)blockIdx.x < nplace) align_place_fused_block(pp, blockIdx.x);
  else quant_fp8_group128_block<DT>(q, (int64_t)blockIdx.x - nplace);
}

}  // namespace
}  // namespace dlb

extern "C" size_t dlb_moe_align_ws_bytes(int64_t numel, int E) {
  if (numel < 0 || E < 1) return 0;
  return (size_t)dlb::num_chunks(numel) * (size_t)E * sizeof(int32_t);
}

namespace dlb {
namespace {

// argument checks shared by the two alignment entry points (everything but the scratch)
int check_align_args(const void* topk_ids, int64_t numel, int E, int block,
                     const int32_t* sorted_ids, int64_t sorted_cap, const int32_t* expert_ids,
                     int64_t expert_ids_cap, const int32_t* num_post_pad) {
  if (numel < 0 || E < 1 || block < 1) return DLB_ERR_BAD_ARG;
  if (E > kMaxE) return DLB_ERR_UNSUPPORTED;
  if (numel + (int64_t)E * block >= (int64_t)0x7fffffff) return DLB_ERR_UNSUPPORTED;
  if (!sorted_ids || !expert_ids || !num_post_pad || (numel > 0 && !topk_ids))
    return DLB_ERR_BAD_ARG;
  if (sorted_cap < numel + (int64_t)E * (block - 1)) return DLB_ERR_BAD_ARG;
  if (expert_ids_cap < ceil_div(sorted_cap, block)) return DLB_ERR_BAD_ARG;
  return DLB_OK;
}

// the launches of the alignment; chunk_counts holds num_chunks(numel) x E int32, every word of
// which the counting pass overwrites before anything reads it (nothing has to start at zero)
int launch_align(const IdxArray topk_ids, int64_t numel, int E, int block, int32_t* sorted_ids,
                 int64_t sorted_cap, int32_t* expert_ids, int64_t expert_ids_cap, int32_t* counts,
                 int32_t* num_post_pad, int32_t* chunk_counts, hipStream_t s,
                 const QuantParams* quant = nullptr, int quant_dtype = DLB_DTYPE_BF16) {
  const int64_t chunks = num_chunks(numel);
  const int chunk_ids = chunk_ids_for(numel);
  hipLaunchKernelGGL(align_count_kernel, dim3((uint32_t)chunks), dim3(kThreads), 0, s, topk_ids,
                     numel, E, chunk_ids, chunk_counts);
  if (chunks <= kFusedChunks) {
    // (with numel = 0 the single chunk is empty: the extra workgroup still writes pads, tails and totals)
    const PlaceParams pp = {topk_ids,   numel,      E,          block,          chunk_counts, (int)chunks,
                            chunk_ids,  sorted_ids, sorted_cap, expert_ids,     expert_ids_cap,
                            counts,     num_post_pad};
    if (quant && quant->total_groups > 0) {
      const uint32_t grid = (uint32_t)(chunks + 1 + ceil_div(quant->total_groups, kQuantGroupsPerBlock));
      if (quant_dtype == DLB_DTYPE_BF16)
        hipLaunchKernelGGL(align_place_quant_kernel<DLB_DTYPE_BF16>, dim3(grid), dim3(kThreads), 0, s, pp, *quant);
      else
        hipLaunchKernelGGL(align_place_quant_kernel<DLB_DTYPE_F16>, dim3(grid), dim3(kThreads), 0, s, pp, *quant);
    } else {
      hipLaunchKernelGGL(align_place_fused_kernel, dim3((uint32_t)chunks + 1), dim3(kThreads), 0, s, pp);
    }
    return launch_status();
  }
  if (quant) return DLB_ERR_UNSUPPORTED;  // (the caller launches the quantiser on its own then)
  hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, chunk_counts, chunks, E, block,
                     (int32_t)numel, sorted_ids, sorted_cap, expert_ids, expert_ids_cap, counts,
                     num_post_pad);
  if (numel > 0)
    hipLaunchKernelGGL(align_place_kernel, dim3((uint32_t)chunks), dim3(kThreads), 0, s, topk_ids,
                       numel, E, chunk_counts, sorted_ids);
  return launch_status();
}

// ---- scratch of the entry point that allocates nothing --------------------------------------
// The per-chunk count table of up to kStaticChunks chunks x kMaxE experts (256 KB) lives in a
// file-scope device array: every GPU the library runs on holds one copy of it until the process
// ends.  In host code the array's name is only a handle, not a device address; the address on
// the current device comes from hipGetSymbolAddress, once per device, and is what the kernels
// receive.
constexpr int kStaticChunks = kFusedChunks;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) int32_t scratch[kStaticChunks * kMaxE];

std::mutex scratch_mutex;
int32_t* scratch_ptr[kMaxDevices];  // per device, filled on the first call made on that device

int static_scratch(int32_t** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return DLB_ERR_LAUNCH;
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return DLB_ERR_LAUNCH;
    }
    scratch_ptr[dev] = (int32_t*)ptr;
  }
  *out = scratch_ptr[dev];
  return DLB_OK;
}

}  // namespace
}  // namespace dlb

extern "C" int dlb_moe_align_block_size(const void* topk_ids, int ids_int64, int64_t numel, int E, int block,
                                        int32_t* sorted_ids, int64_t sorted_cap,
                                        int32_t* expert_ids, int64_t expert_ids_cap,
                                        int32_t* counts, int32_t* num_post_pad, void* ws,
                                        size_t ws_bytes, void* stream) {
  using namespace dlb;
  const int st = check_align_args(topk_ids, numel, E, block, sorted_ids, sorted_cap, expert_ids,
                                  expert_ids_cap, num_post_pad);
  if (st != DLB_OK) return st;
  if (!ws || ws_bytes < dlb_moe_align_ws_bytes(numel, E)) return DLB_ERR_WORKSPACE;
  return launch_align(idx_array(topk_ids, ids_int64 ? 1 : 0, 0), numel, E, block, sorted_ids, sorted_cap,
                      expert_ids, expert_ids_cap, counts, num_post_pad, (int32_t*)ws,
                      (hipStream_t)stream);
}

extern "C" int dlb_moe_align_quant_fp8(const void* topk_ids, int ids_int64, int64_t numel, int E, int block,
                                       int32_t* sorted_ids, int64_t sorted_cap,
                                       int32_t* expert_ids, int64_t expert_ids_cap,
                                       int32_t* counts, int32_t* num_post_pad, void* ws,
                                       size_t ws_bytes, const void* x, void* xq, float* xs,
                                       int64_t M, int K, int64_t ld_x, int64_t ld_q, int64_t ld_s,
                                       int dtype, void* stream) {
  using namespace dlb;
  const int st = check_align_args(topk_ids, numel, E, block, sorted_ids, sorted_cap, expert_ids,
                                  expert_ids_cap, num_post_pad);
  if (st != DLB_OK) return st;
  if (!ws || ws_bytes < dlb_moe_align_ws_bytes(numel, E)) return DLB_ERR_WORKSPACE;
  QuantParams q;
  const int sq = fill_quant_params(q, x, xq, xs, M, K, ld_x, ld_q, ld_s, dtype);
  if (sq != DLB_OK) return sq;
  const IdxArray ids = idx_array(topk_ids, ids_int64 ? 1 : 0, 0);
  if (num_chunks(numel) <= kFusedChunks)
    return launch_align(ids, numel, E, block, sorted_ids, sorted_cap, expert_ids,
                        expert_ids_cap, counts, num_post_pad, (int32_t*)ws, (hipStream_t)stream, &q,
                        dtype);
  // more routing slots than the fused placement takes: the separate launches
  const int sa = launch_align(ids, numel, E, block, sorted_ids, sorted_cap, expert_ids,
                              expert_ids_cap, counts, num_post_pad, (int32_t*)ws, (hipStream_t)stream);
  if (sa != DLB_OK) return sa;
  return dlb_per_token_group_quant_fp8(x, xq, xs, M, K, ld_x, ld_q, ld_s, dtype, stream);
}

extern "C" int64_t dlb_moe_align_block_size_static_max_numel(void) {
  return (int64_t)dlb::kStaticChunks * dlb::kChunk;  // = kFusedChunks chunks of the largest size
}

extern "C" int dlb_moe_align_block_size_static(const void* topk_ids, int ids_int64, int64_t numel,
                                               int E, int block, int32_t* sorted_ids, int64_t sorted_cap,
                                               int32_t* expert_ids, int64_t expert_ids_cap,
                                               int32_t* counts, int32_t* num_post_pad,
                                               void* stream) {
  using namespace dlb;
  const int st = check_align_args(topk_ids, numel, E, block, sorted_ids, sorted_cap, expert_ids,
                                  expert_ids_cap, num_post_pad);
  if (st != DLB_OK) return st;
  // the static table holds kStaticChunks chunks: larger inputs must bring their own workspace
  if (numel > dlb_moe_align_block_size_static_max_numel()) return DLB_ERR_WORKSPACE;
  int32_t* chunk_counts = nullptr;
  const int sp = static_scratch(&chunk_counts);
  if (sp != DLB_OK) return sp;
  return launch_align(idx_array(topk_ids, ids_int64 ? 1 : 0, 0), numel, E, block, sorted_ids, sorted_cap,
                      expert_ids, expert_ids_cap, counts, num_post_pad, chunk_counts,
                      (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------
// Router and alignment as one pipeline of two launches: the router kernel also writes the
// per-chunk expert counts (a chunk = the K routing slots of route_chunk_tokens(T) consecutive
// tokens), so the alignment's own counting pass over the ids is not needed.
// ---------------------------------------------------------------------------------------
extern "C" size_t dlb_moe_topk_softmax_align_ws_bytes(int64_t T, int E) {
  if (T < 0 || E < 1) return 0;
  const int64_t chunks = T > 0 ? dlb::ceil_div(T, dlb::route_chunk_tokens(T)) : 1;
  return (size_t)chunks * (size_t)E * sizeof(int32_t);
}

extern "C" int dlb_moe_topk_softmax_align_f32(const void* logits, float* weights, int32_t* ids,
                                              int64_t T, int E, int K, int64_t ld_logits,
                                              int logits_dtype, int renormalize, int block,
                                              int32_t* sorted_ids,
                                              int64_t sorted_cap, int32_t* expert_ids,
                                              int64_t expert_ids_cap, int32_t* counts,
                                              int32_t* num_post_pad, void* ws, size_t ws_bytes,
                                              void* stream) {
  using namespace dlb;
  if (T < 0 || E < 1 || K < 1 || K > E || ld_logits < E || block < 1) return DLB_ERR_BAD_ARG;
  if (K > 16 || E > kMaxE) return DLB_ERR_UNSUPPORTED;
  if (logits_dtype != DLB_DTYPE_F32 && logits_dtype != DLB_DTYPE_BF16 && logits_dtype != DLB_DTYPE_F16)
    return DLB_ERR_UNSUPPORTED;
  const int64_t numel = T * K;
  if (numel + (int64_t)E * block >= (int64_t)0x7fffffff) return DLB_ERR_UNSUPPORTED;
  const int chunk_tokens = route_chunk_tokens(T);
  const int64_t chunks = T > 0 ? ceil_div(T, chunk_tokens) : 1;
  // larger inputs take the two separate entry points (their scan runs as its own launch)
  if (chunks > kFusedChunks) return DLB_ERR_UNSUPPORTED;
  if (!sorted_ids || !expert_ids || !num_post_pad || (T > 0 && (!logits || !weights || !ids)))
    return DLB_ERR_BAD_ARG;
  if (sorted_cap < numel + (int64_t)E * (block - 1)) return DLB_ERR_BAD_ARG;
  if (expert_ids_cap < ceil_div(sorted_cap, block)) return DLB_ERR_BAD_ARG;
  if (!ws || ws_bytes < dlb_moe_topk_softmax_align_ws_bytes(T, E)) return DLB_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  int32_t* chunk_counts = (int32_t*)ws;
  if (T > 0) {
    const int st = launch_topk_softmax_count(logits, logits_dtype, weights, ids, T, E, K, ld_logits,
                                             renormalize, chunk_tokens, chunk_counts, s);
    if (st != DLB_OK) return st;
  } else {
    // no tokens: the single chunk is empty, but its row of the table is still read
    hipLaunchKernelGGL(align_count_kernel, dim3(1), dim3(kThreads), 0, s, IdxArray{ids, 0}, (int64_t)0, E,
                       kChunk, chunk_counts);
  }
  const PlaceParams pp = {IdxArray{ids, 0}, numel, E, block, chunk_counts, (int)chunks,
                          chunk_tokens * K, sorted_ids, sorted_cap, expert_ids, expert_ids_cap,
                          counts,     num_post_pad};
  hipLaunchKernelGGL(align_place_fused_kernel, dim3((uint32_t)chunks + 1), dim3(kThreads), 0, s, pp);
  return launch_status();
}
