// Memory-bound decoder-layer helpers for gfx950 that sit either side of the attention and MoE
// kernels: KV-cache fill, RMSNorm (+ residual add) and rotary position embedding.
//
//  * fill_kv_cache   python/dlBLAS/dlblas/kernels/fill_kv_cache.py:23-185  (paged cache scatter)
//  * rms_norm        python/dlBLAS/dlblas/kernels/rms_norm.py:8-133, add_rms_norm.py:9-80
//  * apply_rotary    python/dlBLAS/dlblas/kernels/apply_rotary_pos_emb.py:8-164
//
// All three are pure HBM streams; each lane moves 128-bit vectors and a workgroup owns a
// token row, so every access is a full, contiguous cache line.
#include "common.h"

namespace dlb {
namespace {

// ---------------------------------------------------------------------------------------
// fill_kv_cache: token t of sequence b (its i-th new token) goes to cache position
// history_b + i, i.e. page block_offsets[b][pos / page], slot pos % page.  One wavefront per
// new token; rows are copied as bytes in 16-byte chunks (H * D * elem bytes per token).
// ---------------------------------------------------------------------------------------
struct FillParams {
  const unsigned char* ks;
  const unsigned char* vs;
  unsigned char* kc;
  unsigned char* vc;
  IdxArray q_start;
  IdxArray q_len;
  IdxArray kv_len;
  IdxArray block_table;
  int64_t ks_tok, ks_head, vs_tok, vs_head;              // bytes
  int64_t kc_page, kc_slot, kc_head, vc_page, vc_slot, vc_head;  // bytes
  int64_t bt_stride;
  int64_t num_tokens;
  int batch, heads, page, max_blocks;
  int k_row_bytes, v_row_bytes;  // head_dim * elem, head_dim_v * elem
  int vec;                       // 1: 16-byte chunks, 0: single bytes
};

constexpr int kFillTokens = 1;  // tokens (= wavefronts) per workgroup; 2 and 4 measured 1.5 % and 3.7 % slower

// One wavefront per new token: it finds the sequence that owns the token with a ballot over
// the batch, then streams the token's K and V rows into the page slot (no barriers).
__global__ __launch_bounds__(64 * kFillTokens) void fill_kv_cache_kernel(const FillParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * kFillTokens + (threadIdx.x >> 6);
  if (t >= p.num_tokens) return;
  int b = -1;
  for (int b0 = 0; b0 < p.batch && b < 0; b0 += 64) {
    const int bb = b0 + lane;
    bool hit = false;
    if (bb < p.batch) {
      const int s0 = p.q_start[bb], n = p.q_len[bb];
      hit = t >= s0 && t < (int64_t)s0 + n;
    }
    const uint64_t m = __ballot(hit);
    if (m) b = b0 + __builtin_ctzll(m);  // sequences do not overlap: at most one owner
  }
  if (b < 0) return;
  const int i = (int)(t - p.q_start[b]);
  const int pos = p.kv_len[b] - p.q_len[b] + i;
  const int pi = pos / p.page;
  if (pos < 0 || pi >= p.max_blocks) return;
  const int64_t pg = p.block_table[(int64_t)b * p.bt_stride + pi];
  const int slot = pos - pi * p.page;

  const unsigned char* ksrc = p.ks + t * p.ks_tok;
  const unsigned char* vsrc = p.vs + t * p.vs_tok;
  unsigned char* kdst = p.kc + pg * p.kc_page + (int64_t)slot * p.kc_slot;
  unsigned char* vdst = p.vc + pg * p.vc_page + (int64_t)slot * p.vc_slot;
  if (p.vec) {
    const int kc_per_head = p.k_row_bytes >> 4, vc_per_head = p.v_row_bytes >> 4;
    for (int u = lane; u < p.heads * kc_per_head; u += 64) {
      const int h = u / kc_per_head, c = u - h * kc_per_head;
      __builtin_nontemporal_store(__builtin_nontemporal_load((const u32x4*)(ksrc + h * p.ks_head + c * 16)),
                                  (u32x4*)(kdst + h * p.kc_head + c * 16));
    }
    for (int u = lane; u < p.heads * vc_per_head; u += 64) {
      const int h = u / vc_per_head, c = u - h * vc_per_head;
      __builtin_nontemporal_store(__builtin_nontemporal_load((const u32x4*)(vsrc + h * p.vs_head + c * 16)),
                                  (u32x4*)(vdst + h * p.vc_head + c * 16));
    }
  } else {
    for (int u = lane; u < p.heads * p.k_row_bytes; u += 64) {
      const int h = u / p.k_row_bytes, c = u - h * p.k_row_bytes;
      kdst[h * p.kc_head + c] = ksrc[h * p.ks_head + c];
    }
    for (int u = lane; u < p.heads * p.v_row_bytes; u += 64) {
      const int h = u / p.v_row_bytes, c = u - h * p.v_row_bytes;
      vdst[h * p.vc_head + c] = vsrc[h * p.vs_head + c];
    }
  }
}

// ---------------------------------------------------------------------------------------
// rms_norm: out = weight * round(x * rsqrt(mean(x^2) + eps)), optionally on x = round(x + res)
// with the sum written to out_residual.  One workgroup per row; the row lives in registers
// (up to kMaxVec 128-bit vectors per thread) so it is read once.
// ---------------------------------------------------------------------------------------
constexpr int kNormThreads = 256;
constexpr int kMaxVec = 8;  // 256 threads * 8 vectors * 8 elements = 16384 columns

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.0f;
#pragma unroll
  for (int w = 0; w < kNormThreads / 64; ++w) s += red[w];
  return s;
}

template <int DT, bool ADD>
__global__ __launch_bounds__(kNormThreads) void rms_norm_kernel(
    const unsigned short* __restrict__ x, const unsigned short* __restrict__ w,
    const unsigned short* __restrict__ res, unsigned short* __restrict__ out,
    unsigned short* __restrict__ out_res, int N, int64_t ld_x, int64_t ld_res, int64_t ld_out,
    int64_t ld_out_res, float eps) {
  __shared__ float red[kNormThreads / 64];
  const int64_t row = blockIdx.x;
  const int nvec = N >> 3;
  u32x4 v[kMaxVec];
  float ss = 0.0f;
#pragma unroll
  for (int q = 0; q < kMaxVec; ++q) {
    const int i = q * kNormThreads + threadIdx.x;
    if (i < nvec) {
      v[q] = __builtin_nontemporal_load((const u32x4*)(x + row * ld_x + 8 * i));  // streamed once
      if (ADD) {
        const u32x4 r = __builtin_nontemporal_load((const u32x4*)(res + row * ld_res + 8 * i));
#pragma unroll
        for (int k = 0; k < 4; ++k)
          v[q][k] = Elem<DT>::pack(Elem<DT>::lo(v[q][k]) + Elem<DT>::lo(r[k]),
                                   Elem<DT>::hi(v[q][k]) + Elem<DT>::hi(r[k]));
        __builtin_nontemporal_store(v[q], (u32x4*)(out_res + row * ld_out_res + 8 * i));
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float a = Elem<DT>::lo(v[q][k]), b = Elem<DT>::hi(v[q][k]);
        ss += a * a + b * b;
      }
    }
  }
  const float var = block_sum(ss, red) / (float)N;
  const float inv = rsqrtf(var + eps);
#pragma unroll
  for (int q = 0; q < kMaxVec; ++q) {
    const int i = q * kNormThreads + threadIdx.x;
    if (i < nvec) {
      const u32x4 wv = *(const u32x4*)(w + 8 * i);
      u32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        // normalised value rounded to the storage type, then times the weight, rounded again
        const unsigned int nrm = Elem<DT>::pack(Elem<DT>::lo(v[q][k]) * inv, Elem<DT>::hi(v[q][k]) * inv);
        o[k] = Elem<DT>::pack(Elem<DT>::lo(nrm) * Elem<DT>::lo(wv[k]),
                              Elem<DT>::hi(nrm) * Elem<DT>::hi(wv[k]));
      }
      __builtin_nontemporal_store(o, (u32x4*)(out + row * ld_out + 8 * i));
    }
  }
}

// fp32 rows: the same kernel shape on four-element vectors (nothing is rounded on the way, so
// the two rounding points above coincide).
constexpr int kMaxVecF32 = 16;  // 256 threads * 16 vectors * 4 elements = 16384 columns
template <bool ADD>
__global__ __launch_bounds__(kNormThreads) void rms_norm_f32_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ res,
    float* __restrict__ out, float* __restrict__ out_res, int N, int64_t ld_x, int64_t ld_res,
    int64_t ld_out, int64_t ld_out_res, float eps) {
  __shared__ float red[kNormThreads / 64];
  const int64_t row = blockIdx.x;
  const int nvec = N >> 2;
  f32x4 v[kMaxVecF32];
  float ss = 0.0f;
#pragma unroll
  for (int q = 0; q < kMaxVecF32; ++q) {
    const int i = q * kNormThreads + threadIdx.x;
    if (i < nvec) {
      v[q] = __builtin_nontemporal_load((const f32x4*)(x + row * ld_x + 4 * i));
      if (ADD) {
        v[q] += __builtin_nontemporal_load((const f32x4*)(res + row * ld_res + 4 * i));
        __builtin_nontemporal_store(v[q], (f32x4*)(out_res + row * ld_out_res + 4 * i));
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) ss += v[q][k] * v[q][k];
    }
  }
  const float var = block_sum(ss, red) / (float)N;
  const float inv = rsqrtf(var + eps);
#pragma unroll
  for (int q = 0; q < kMaxVecF32; ++q) {
    const int i = q * kNormThreads + threadIdx.x;
    if (i < nvec) {
      const f32x4 wv = *(const f32x4*)(w + 4 * i);
      f32x4 o;
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = (v[q][k] * inv) * wv[k];
      __builtin_nontemporal_store(o, (f32x4*)(out + row * ld_out + 4 * i));
    }
  }
}

// ---------------------------------------------------------------------------------------
// rotary: for d < D/2:  out[d]       = x[d] * cos[d]       - x[d + D/2] * sin[d]
//                       out[d + D/2] = x[d + D/2] * cos[d + D/2] + x[d] * sin[d + D/2]
// (x * cos + rotate_half(x) * sin).  One workgroup per token; a thread handles 8 low and the
// 8 matching high elements of one head, reads both before writing, so in-place is allowed.
// ---------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void rotary_kernel(
    const unsigned short* __restrict__ q, const unsigned short* __restrict__ k,
    const unsigned short* __restrict__ cos_, const unsigned short* __restrict__ sin_,
    unsigned short* qo, unsigned short* ko, int Hq, int Hk, int D, int64_t q_st, int64_t q_sh,
    int64_t k_st, int64_t k_sh, int64_t qo_st, int64_t qo_sh, int64_t ko_st, int64_t ko_sh,
    int64_t cs_st) {
  const int64_t t = blockIdx.x;
  const int half = D >> 1;
  const int vec_per_head = half >> 3;
  const int total = (Hq + Hk) * vec_per_head;
  for (int u = threadIdx.x; u < total; u += 256) {
    const int h = u / vec_per_head, c = u - h * vec_per_head;
    const unsigned short* src;
    unsigned short* dst;
    if (h < Hq) {
      src = q + t * q_st + (int64_t)h * q_sh;
      dst = qo + t * qo_st + (int64_t)h * qo_sh;
    } else {
      src = k + t * k_st + (int64_t)(h - Hq) * k_sh;
      dst = ko + t * ko_st + (int64_t)(h - Hq) * ko_sh;
    }
    // q/k are streamed once (non-temporal); cos/sin are shared by every head of the token
    const u32x4 xl = __builtin_nontemporal_load((const u32x4*)(src + 8 * c));
    const u32x4 xh = __builtin_nontemporal_load((const u32x4*)(src + half + 8 * c));
    const u32x4 cl = *(const u32x4*)(cos_ + t * cs_st + 8 * c);
    const u32x4 ch = *(const u32x4*)(cos_ + t * cs_st + half + 8 * c);
    const u32x4 sl = *(const u32x4*)(sin_ + t * cs_st + 8 * c);
    const u32x4 sh = *(const u32x4*)(sin_ + t * cs_st + half + 8 * c);
    u32x4 ol, oh;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float l0 = Elem<DT>::lo(xl[j]), l1 = Elem<DT>::hi(xl[j]);
      const float h0 = Elem<DT>::lo(xh[j]), h1 = Elem<DT>::hi(xh[j]);
      ol[j] = Elem<DT>::pack(l0 * Elem<DT>::lo(cl[j]) - h0 * Elem<DT>::lo(sl[j]),
                             l1 * Elem<DT>::hi(cl[j]) - h1 * Elem<DT>::hi(sl[j]));
      oh[j] = Elem<DT>::pack(h0 * Elem<DT>::lo(ch[j]) + l0 * Elem<DT>::lo(sh[j]),
                             h1 * Elem<DT>::hi(ch[j]) + l1 * Elem<DT>::hi(sh[j]));
    }
    __builtin_nontemporal_store(ol, (u32x4*)(dst + 8 * c));
    __builtin_nontemporal_store(oh, (u32x4*)(dst + half + 8 * c));
  }
}

// fp32 tensors: a thread handles 4 low and the 4 matching high elements of one head
__global__ __launch_bounds__(256) void rotary_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ cos_,
    const float* __restrict__ sin_, float* qo, float* ko, int Hq, int Hk, int D, int64_t q_st,
    int64_t q_sh, int64_t k_st, int64_t k_sh, int64_t qo_st, int64_t qo_sh, int64_t ko_st,
    int64_t ko_sh, int64_t cs_st) {
  const int64_t t = blockIdx.x;
  const int half = D >> 1;
  const int vec_per_head = half >> 2;
  const int total = (Hq + Hk) * vec_per_head;
  for (int u = threadIdx.x; u < total; u += 256) {
    const int h = u / vec_per_head, c = u - h * vec_per_head;
    const float* src;
    float* dst;
    if (h < Hq) {
      src = q + t * q_st + (int64_t)h * q_sh;
      dst = qo + t * qo_st + (int64_t)h * qo_sh;
    } else {
      src = k + t * k_st + (int64_t)(h - Hq) * k_sh;
      dst = ko + t * ko_st + (int64_t)(h - Hq) * ko_sh;
    }
    const f32x4 xl = __builtin_nontemporal_load((const f32x4*)(src + 4 * c));
    const f32x4 xh = __builtin_nontemporal_load((const f32x4*)(src + half + 4 * c));
    const f32x4 cl = *(const f32x4*)(cos_ + t * cs_st + 4 * c);
    const f32x4 ch = *(const f32x4*)(cos_ + t * cs_st + half + 4 * c);
    const f32x4 sl = *(const f32x4*)(sin_ + t * cs_st + 4 * c);
    const f32x4 sh = *(const f32x4*)(sin_ + t * cs_st + half + 4 * c);
    f32x4 ol, oh;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ol[j] = xl[j] * cl[j] - xh[j] * sl[j];
      oh[j] = xh[j] * ch[j] + xl[j] * sh[j];
    }
    __builtin_nontemporal_store(ol, (f32x4*)(dst + 4 * c));
    __builtin_nontemporal_store(oh, (f32x4*)(dst + half + 4 * c));
  }
}

// ---------------------------------------------------------------------------------------
// Element-wise variants for shapes the vector kernels do not take: rows of any length and any
// alignment (rms_norm; the reference masks `offsets < N_COLS`, rms_norm.py:8-75) and any even
// head size (rotary).  Same arithmetic and rounding points, one element per thread and step.
// ---------------------------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ float ld_elem(const void* p, int64_t i) {
  if constexpr (DT == DLB_DTYPE_F32) return ((const float*)p)[i];
  else return Elem<DT>::load1(p, i);
}
template <int DT>
__device__ __forceinline__ void st_elem(void* p, int64_t i, float v) {
  if constexpr (DT == DLB_DTYPE_F32) ((float*)p)[i] = v;
  else Elem<DT>::store1(p, i, v);
}
// v rounded to the storage type
template <int DT>
__device__ __forceinline__ float round_elem(float v) {
  if constexpr (DT == DLB_DTYPE_F32) return v;
  else return Elem<DT>::lo(Elem<DT>::pack(v, 0.0f));
}

template <int DT, bool ADD>
__global__ __launch_bounds__(kNormThreads) void rms_norm_any_kernel(
    const void* __restrict__ x, const void* __restrict__ w, const void* __restrict__ res,
    void* __restrict__ out, void* __restrict__ out_res, int N, int64_t ld_x, int64_t ld_res,
    int64_t ld_out, int64_t ld_out_res, float eps) {
  __shared__ float red[kNormThreads / 64];
  const int64_t row = blockIdx.x;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < N; i += kNormThreads) {
    float v = ld_elem<DT>(x, row * ld_x + i);
    if (ADD) {
      v = round_elem<DT>(v + ld_elem<DT>(res, row * ld_res + i));
      st_elem<DT>(out_res, row * ld_out_res + i, v);  // read back below by the thread that wrote it
    }
    ss += v * v;
  }
  const float var = block_sum(ss, red) / (float)N;
  const float inv = rsqrtf(var + eps);
  for (int i = threadIdx.x; i < N; i += kNormThreads) {
    const float v = ADD ? ld_elem<DT>(out_res, row * ld_out_res + i) : ld_elem<DT>(x, row * ld_x + i);
    st_elem<DT>(out, row * ld_out + i, round_elem<DT>(v * inv) * ld_elem<DT>(w, i));
  }
}

template <int DT>
__global__ __launch_bounds__(256) void rotary_any_kernel(
    const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ cos_,
    const void* __restrict__ sin_, void* qo, void* ko, int Hq, int Hk, int D, int64_t q_st,
    int64_t q_sh, int64_t k_st, int64_t k_sh, int64_t qo_st, int64_t qo_sh, int64_t ko_st,
    int64_t ko_sh, int64_t cs_st) {
  const int64_t t = blockIdx.x;
  const int half = D >> 1;
  const int total = (Hq + Hk) * half;
  for (int u = threadIdx.x; u < total; u += 256) {
    const int h = u / half, d = u - h * half;
    const void* src = h < Hq ? q : k;
    void* dst = h < Hq ? qo : ko;
    const int64_t so = h < Hq ? t * q_st + (int64_t)h * q_sh : t * k_st + (int64_t)(h - Hq) * k_sh;
    const int64_t dof = h < Hq ? t * qo_st + (int64_t)h * qo_sh : t * ko_st + (int64_t)(h - Hq) * ko_sh;
    // both halves are read before either is written: in place is allowed
    const float xl = ld_elem<DT>(src, so + d), xh = ld_elem<DT>(src, so + half + d);
    const float cl = ld_elem<DT>(cos_, t * cs_st + d), ch = ld_elem<DT>(cos_, t * cs_st + half + d);
    const float sl = ld_elem<DT>(sin_, t * cs_st + d), sh = ld_elem<DT>(sin_, t * cs_st + half + d);
    st_elem<DT>(dst, dof + d, xl * cl - xh * sl);
    st_elem<DT>(dst, dof + half + d, xh * ch + xl * sh);
  }
}

inline bool mult16(int64_t v) { return (v & 15) == 0; }

}  // namespace
}  // namespace dlb

extern "C" int dlb_fill_kv_cache(const void* k_states, const void* v_states, void* k_cache,
                                 void* v_cache, const void* q_start_loc,
                                 const void* q_seq_len, const void* kv_seq_len,
                                 const void* block_table, int index64_mask, int64_t num_tokens,
                                 int batch,
                                 int heads, int head_dim, int head_dim_v, int page, int max_blocks,
                                 int elem_size, int64_t ks_stride_tok, int64_t ks_stride_head,
                                 int64_t vs_stride_tok, int64_t vs_stride_head,
                                 int64_t kc_stride_page, int64_t kc_stride_slot,
                                 int64_t kc_stride_head, int64_t vc_stride_page,
                                 int64_t vc_stride_slot, int64_t vc_stride_head,
                                 int64_t bt_stride, void* stream) {
  using namespace dlb;
  if (num_tokens < 0 || batch < 0 || heads < 1 || head_dim < 1 || head_dim_v < 1 || page < 1 ||
      max_blocks < 1 || elem_size < 1)
    return DLB_ERR_BAD_ARG;
  if (num_tokens == 0 || batch == 0) return DLB_OK;
  if (!k_states || !v_states || !k_cache || !v_cache || !q_start_loc || !q_seq_len ||
      !kv_seq_len || !block_table)
    return DLB_ERR_BAD_ARG;
  if (num_tokens > 0x7fffffff) return DLB_ERR_UNSUPPORTED;
  FillParams p;
  const int64_t es = elem_size;
  p.ks = (const unsigned char*)k_states;
  p.vs = (const unsigned char*)v_states;
  p.kc = (unsigned char*)k_cache;
  p.vc = (unsigned char*)v_cache;
  if (index64_mask & ~15) return DLB_ERR_BAD_ARG;
  p.q_start = idx_array(q_start_loc, index64_mask, 0);
  p.q_len = idx_array(q_seq_len, index64_mask, 1);
  p.kv_len = idx_array(kv_seq_len, index64_mask, 2);
  p.block_table = idx_array(block_table, index64_mask, 3);
  p.ks_tok = ks_stride_tok * es;
  p.ks_head = ks_stride_head * es;
  p.vs_tok = vs_stride_tok * es;
  p.vs_head = vs_stride_head * es;
  p.kc_page = kc_stride_page * es;
  p.kc_slot = kc_stride_slot * es;
  p.kc_head = kc_stride_head * es;
  p.vc_page = vc_stride_page * es;
  p.vc_slot = vc_stride_slot * es;
  p.vc_head = vc_stride_head * es;
  p.bt_stride = bt_stride;
  p.batch = batch;
  p.num_tokens = num_tokens;
  p.heads = heads;
  p.page = page;
  p.max_blocks = max_blocks;
  p.k_row_bytes = head_dim * elem_size;
  p.v_row_bytes = head_dim_v * elem_size;
  p.vec = aligned16(k_states) && aligned16(v_states) && aligned16(k_cache) && aligned16(v_cache) &&
          mult16(p.k_row_bytes) && mult16(p.v_row_bytes) && mult16(p.ks_tok) && mult16(p.ks_head) &&
          mult16(p.vs_tok) && mult16(p.vs_head) && mult16(p.kc_page) && mult16(p.kc_slot) &&
          mult16(p.kc_head) && mult16(p.vc_page) && mult16(p.vc_slot) && mult16(p.vc_head);
  hipLaunchKernelGGL(fill_kv_cache_kernel, dim3((uint32_t)ceil_div(num_tokens, kFillTokens)),
                     dim3(64 * kFillTokens), 0, (hipStream_t)stream, p);
  return launch_status();
}

extern "C" int dlb_rms_norm(const void* x, const void* weight, const void* residual, void* out,
                            void* out_residual, int64_t M, int N, int64_t ld_x, int64_t ld_res,
                            int64_t ld_out, int64_t ld_out_res, float eps, int dtype,
                            void* stream) {
  using namespace dlb;
  if (M < 0 || N < 1) return DLB_ERR_BAD_ARG;
  if (M == 0) return DLB_OK;
  if (!x || !weight || !out || (residual && !out_residual)) return DLB_ERR_BAD_ARG;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16 && dtype != DLB_DTYPE_F32)
    return DLB_ERR_UNSUPPORTED;
  const int vec = dtype == DLB_DTYPE_F32 ? 4 : 8;  // elements per 16-byte vector
  if (ld_x < N || ld_out < N || (residual && (ld_res < N || ld_out_res < N))) return DLB_ERR_BAD_ARG;
  if (M > 0x7fffffff) return DLB_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)M), block(kNormThreads);
  // the vector kernels keep a row of up to 16384 elements in registers and move 16-byte pieces;
  // any other row length or alignment takes the element-wise kernel
  bool vector_ok = N % vec == 0 && N <= kNormThreads * kMaxVec * 8 && ld_x % vec == 0 &&
                   ld_out % vec == 0 && aligned16(x) && aligned16(weight) && aligned16(out);
  if (residual)
    vector_ok = vector_ok && ld_res % vec == 0 && ld_out_res % vec == 0 && aligned16(residual) &&
                aligned16(out_residual);
  if (!vector_ok) {
#define DLB_LAUNCH_NORM_ANY(DT_)                                                                   \
  do {                                                                                             \
    if (residual)                                                                                  \
      hipLaunchKernelGGL((rms_norm_any_kernel<DT_, true>), grid, block, 0, s, x, weight, residual, \
                         out, out_residual, N, ld_x, ld_res, ld_out, ld_out_res, eps);             \
    else                                                                                           \
      hipLaunchKernelGGL((rms_norm_any_kernel<DT_, false>), grid, block, 0, s, x, weight, residual, \
                         out, out_residual, N, ld_x, ld_res, ld_out, ld_out_res, eps);             \
  } while (0)
    if (dtype == DLB_DTYPE_F32) DLB_LAUNCH_NORM_ANY(DLB_DTYPE_F32);
    else if (dtype == DLB_DTYPE_BF16) DLB_LAUNCH_NORM_ANY(DLB_DTYPE_BF16);
    else DLB_LAUNCH_NORM_ANY(DLB_DTYPE_F16);
#undef DLB_LAUNCH_NORM_ANY
    return launch_status();
  }
  static_assert(kMaxVecF32 * 4 == kMaxVec * 8, "same row length limit for every element type");
  if (dtype == DLB_DTYPE_F32) {
    if (residual)
      hipLaunchKernelGGL(rms_norm_f32_kernel<true>, grid, block, 0, s, (const float*)x,
                         (const float*)weight, (const float*)residual, (float*)out,
                         (float*)out_residual, N, ld_x, ld_res, ld_out, ld_out_res, eps);
    else
      hipLaunchKernelGGL(rms_norm_f32_kernel<false>, grid, block, 0, s, (const float*)x,
                         (const float*)weight, (const float*)residual, (float*)out,
                         (float*)out_residual, N, ld_x, ld_res, ld_out, ld_out_res, eps);
    return launch_status();
  }
#define DLB_LAUNCH_NORM(DT_, ADD_)                                                            \
  hipLaunchKernelGGL((rms_norm_kernel<DT_, ADD_>), grid, block, 0, s, (const unsigned short*)x, \
                     (const unsigned short*)weight, (const unsigned short*)residual,          \
                     (unsigned short*)out, (unsigned short*)out_residual, N, ld_x, ld_res,    \
                     ld_out, ld_out_res, eps)
  if (dtype == DLB_DTYPE_BF16) {
    if (residual) DLB_LAUNCH_NORM(DLB_DTYPE_BF16, true);
    else DLB_LAUNCH_NORM(DLB_DTYPE_BF16, false);
  } else {
    if (residual) DLB_LAUNCH_NORM(DLB_DTYPE_F16, true);
    else DLB_LAUNCH_NORM(DLB_DTYPE_F16, false);
  }
#undef DLB_LAUNCH_NORM
  return launch_status();
}

extern "C" int dlb_apply_rotary_pos_emb(const void* q, const void* k, const void* cos,
                                        const void* sin, void* q_out, void* k_out,
                                        int64_t num_tokens, int Hq, int Hk, int D,
                                        int64_t q_stride_tok, int64_t q_stride_head,
                                        int64_t k_stride_tok, int64_t k_stride_head,
                                        int64_t qo_stride_tok, int64_t qo_stride_head,
                                        int64_t ko_stride_tok, int64_t ko_stride_head,
                                        int64_t cs_stride_tok, int dtype, void* stream) {
  using namespace dlb;
  if (num_tokens < 0 || Hq < 0 || Hk < 0 || D < 2) return DLB_ERR_BAD_ARG;
  if (num_tokens == 0 || Hq + Hk == 0) return DLB_OK;
  if (!q || !k || !cos || !sin || !q_out || !k_out) return DLB_ERR_BAD_ARG;
  if (dtype != DLB_DTYPE_BF16 && dtype != DLB_DTYPE_F16 && dtype != DLB_DTYPE_F32)
    return DLB_ERR_UNSUPPORTED;
  const int vec = dtype == DLB_DTYPE_F32 ? 4 : 8;  // elements per 16-byte vector
  if (D % 2 != 0 || num_tokens > 0x7fffffff) return DLB_ERR_UNSUPPORTED;
  const int64_t strides[] = {q_stride_tok,  q_stride_head,  k_stride_tok,  k_stride_head, qo_stride_tok,
                             qo_stride_head, ko_stride_tok, ko_stride_head, cs_stride_tok};
  bool vector_ok = D % (2 * vec) == 0 && aligned16(q) && aligned16(k) && aligned16(cos) &&
                   aligned16(sin) && aligned16(q_out) && aligned16(k_out);
  for (int64_t sd : strides) vector_ok = vector_ok && sd % vec == 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)num_tokens), block(256);
  if (!vector_ok) {  // any even head size, any strides: one element pair per thread and step
#define DLB_LAUNCH_ROTARY_ANY(DT_)                                                               \
  hipLaunchKernelGGL(rotary_any_kernel<DT_>, grid, block, 0, s, q, k, cos, sin, q_out, k_out, Hq, \
                     Hk, D, q_stride_tok, q_stride_head, k_stride_tok, k_stride_head,            \
                     qo_stride_tok, qo_stride_head, ko_stride_tok, ko_stride_head, cs_stride_tok)
    if (dtype == DLB_DTYPE_F32) DLB_LAUNCH_ROTARY_ANY(DLB_DTYPE_F32);
    else if (dtype == DLB_DTYPE_BF16) DLB_LAUNCH_ROTARY_ANY(DLB_DTYPE_BF16);
    else DLB_LAUNCH_ROTARY_ANY(DLB_DTYPE_F16);
#undef DLB_LAUNCH_ROTARY_ANY
    return launch_status();
  }
  if (dtype == DLB_DTYPE_F32)
    hipLaunchKernelGGL(rotary_f32_kernel, grid, block, 0, s, (const float*)q, (const float*)k,
                       (const float*)cos, (const float*)sin, (float*)q_out, (float*)k_out, Hq, Hk,
                       D, q_stride_tok, q_stride_head, k_stride_tok, k_stride_head, qo_stride_tok,
                       qo_stride_head, ko_stride_tok, ko_stride_head, cs_stride_tok);
  else if (dtype == DLB_DTYPE_BF16)
    hipLaunchKernelGGL(rotary_kernel<DLB_DTYPE_BF16>, grid, block, 0, s, (const unsigned short*)q,
                       (const unsigned short*)k, (const unsigned short*)cos,
                       (const unsigned short*)sin, (unsigned short*)q_out, (unsigned short*)k_out,
                       Hq, Hk, D, q_stride_tok, q_stride_head, k_stride_tok, k_stride_head,
                       qo_stride_tok, qo_stride_head, ko_stride_tok, ko_stride_head, cs_stride_tok);
  else
    hipLaunchKernelGGL(rotary_kernel<DLB_DTYPE_F16>, grid, block, 0, s, (const unsigned short*)q,
                       (const unsigned short*)k, (const unsigned short*)cos,
                       (const unsigned short*)sin, (unsigned short*)q_out, (unsigned short*)k_out,
                       Hq, Hk, D, q_stride_tok, q_stride_head, k_stride_tok, k_stride_head,
                       qo_stride_tok, qo_stride_head, ko_stride_tok, ko_stride_head, cs_stride_tok);
  return launch_status();
}
