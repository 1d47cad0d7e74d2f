// Shared device/host helpers for the gfx950 kernels of libdlblas_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/dlblas_hip.h"

namespace dlb {

constexpr int kWave = 64;  // CDNA wavefront width

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

// ---- bf16 / f16 <-> f32 scalar conversions on raw 16-bit patterns -----------------------
__device__ __forceinline__ float bf16_bits_to_f32(unsigned int b) {
  return __uint_as_float(b << 16);
}
// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ unsigned int f32_to_bf16_bits(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float f16_bits_to_f32(unsigned int b) {
  _Float16 h = __builtin_bit_cast(_Float16, (unsigned short)b);
  return (float)h;
}
__device__ __forceinline__ unsigned int f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32: RNE
  return (unsigned int)__builtin_bit_cast(unsigned short, h);
}

template <int DT>
struct Elem;
template <>
struct Elem<DLB_DTYPE_BF16> {
  static __device__ __forceinline__ float lo(unsigned int w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(unsigned int w) {
    return __uint_as_float(w & 0xffff0000u);
  }
  // two floats -> two bf16 in one word: v_cvt_pk_bf16_f32 (round to nearest even, NaN quiet)
  static __device__ __forceinline__ unsigned int pack(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) __bf16 b2;
    const f2 f = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, b2));
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) {
    return bf16_bits_to_f32(((const unsigned short*)p)[i]);
  }
  static __device__ __forceinline__ void store1(void* p, int64_t i, float v) {
    ((unsigned short*)p)[i] = (unsigned short)f32_to_bf16_bits(v);
  }
};
template <>
struct Elem<DLB_DTYPE_F16> {
  static __device__ __forceinline__ float lo(unsigned int w) { return f16_bits_to_f32(w & 0xffffu); }
  static __device__ __forceinline__ float hi(unsigned int w) { return f16_bits_to_f32(w >> 16); }
  static __device__ __forceinline__ unsigned int pack(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f2;
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    const f2 f = {a, b};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(f, h2));
  }
  static __device__ __forceinline__ float load1(const void* p, int64_t i) {
    return f16_bits_to_f32(((const unsigned short*)p)[i]);
  }
  static __device__ __forceinline__ void store1(void* p, int64_t i, float v) {
    ((unsigned short*)p)[i] = (unsigned short)f32_to_f16_bits(v);
  }
};

// ---- DPP cross-lane moves within a row of 16 lanes ---------------------------------------
// dpp_ctrl encodings (GCN3+/CDNA): quad_perm = 0x00..0xff, row_mirror = 0x140,
// row_half_mirror = 0x141.
constexpr int kDppQuadXor1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ unsigned int dpp_u32(unsigned int v) {
  return (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}

// all-reduce over each aligned group of 16 lanes (a DPP row); every lane gets the result.
// After the two quad steps all lanes of a quad agree, so the mirror steps (i <-> 7-i,
// i <-> 15-i) complete a butterfly for any commutative, associative, idempotent-or-not op:
// each step combines two disjoint halves whose members already hold their half's result.
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f32<kDppQuadXor1>(v));
  v = fmaxf(v, dpp_f32<kDppQuadXor2>(v));
  v = fmaxf(v, dpp_f32<kDppRowHalfMirror>(v));
  v = fmaxf(v, dpp_f32<kDppRowMirror>(v));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<kDppQuadXor1>(v);
  v += dpp_f32<kDppQuadXor2>(v);
  v += dpp_f32<kDppRowHalfMirror>(v);
  v += dpp_f32<kDppRowMirror>(v);
  return v;
}

// inclusive prefix sum over the 64 lanes of a wave with DPP moves only (shifts inside each row
// of 16 lanes, then the row totals broadcast to the rows after them): no LDS round trips and no
// per-lane address registers, which a shuffle-based scan keeps live across the whole kernel
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2, 3
  return v;
}

// a pointer the caller knows to be wave-uniform, moved into scalar registers
__device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (const unsigned char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
// wave-uniform LDS byte address of a pointer into __shared__ memory, in a scalar register
__device__ __forceinline__ unsigned int lds_addr(const void* p) {
  typedef const __attribute__((address_space(3))) void* lds_ptr_t;
  return (unsigned int)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(lds_ptr_t)p);
}
// Direct global -> LDS copy of 16 bytes per lane: lane l's bytes land at lds_base + 16 * l
// (lds_base: wave-uniform LDS byte address).  Issued through inline assembly rather than
// __builtin_amdgcn_global_load_lds because the compiler's wait-count pass models the builtin as
// a FLAT access that may complete out of order with LDS reads: while one is in flight every
// LDS wait it inserts becomes lgkmcnt(0), which serialises a pipelined ds_read -> MFMA stream.
// The copy is counted by vmcnt like any other vector load (loads return in order); the compiler
// does not see it, so the caller waits for it explicitly (s_waitcnt vmcnt) before the barrier
// that publishes the data.  Waits the compiler inserts for its own loads stay correct: an
// unseen load that is older completes first, one that is younger only makes the wait longer.
// The helpers write m0 and say so in their clobber lists, so the compiler never keeps a live
// value of its own (an LDS-direct or indexed-register base) in m0 across one of them.
__device__ __forceinline__ void dma16_global_to_lds(const void* gsrc, unsigned int lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(__builtin_amdgcn_readfirstlane((int)lds_base))
               : "memory", "m0");
}

// same copy, addressed as a wave-uniform 64-bit base (scalar registers) plus a 32-bit lane offset
__device__ __forceinline__ void dma16_global_to_lds(const void* sbase, unsigned int voff,
                                                    unsigned int lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane((int)lds_base))
               : "memory", "m0");
}

// the 4-byte form: lane l's dword lands at lds_base + 4 * l
__device__ __forceinline__ void dma4_global_to_lds(const void* gsrc, unsigned int lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :
               : "v"(gsrc), "s"(__builtin_amdgcn_readfirstlane((int)lds_base))
               : "memory", "m0");
}

// the 4-byte form restricted to the lanes of `lane_mask` (a compile-time constant); the other
// lanes neither read nor write
template <unsigned long long lane_mask>
__device__ __forceinline__ void dma4_global_to_lds_masked(const void* gsrc, unsigned int lds_base) {
  unsigned long long saved;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t"
               "global_load_lds_dword %1, off\n\ts_mov_b64 exec, %0"
               : "=&s"(saved)
               : "v"(gsrc), "s"(__builtin_amdgcn_readfirstlane((int)lds_base)), "s"(lane_mask)
               : "memory", "m0");
}

// ds_read_b64_tr_b16: every lane passes the address of four consecutive 16-bit elements; in
// each group of 16 lanes the 16 x 4 elements form a 4-row x 16-column block (row j = lanes
// 4j .. 4j+3 of the group, four columns each) and lane l of the group receives column l,
// rows 0..3, lowest row in the low half of the first register.
__device__ __forceinline__ u32x2 lds_read_tr16(const void* p) {
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p));
}

// the masked 4-byte form addressed as a wave-uniform 64-bit base plus a 32-bit lane offset
template <unsigned long long lane_mask>
__device__ __forceinline__ void dma4_global_to_lds_masked(const void* sbase, unsigned int voff,
                                                          unsigned int lds_base) {
  unsigned long long saved;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
               "global_load_lds_dword %1, %2\n\ts_mov_b64 exec, %0"
               : "=&s"(saved)
               : "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane((int)lds_base)),
                 "s"(lane_mask)
               : "memory", "m0");
}

// max of a value and its partner 32 lanes away (v_permlane32_swap: a register-file exchange,
// no trip through LDS as with ds_bpermute)
__device__ __forceinline__ float max_xor32(float v) {
  typedef __attribute__((ext_vector_type(2))) unsigned int u2;
  const unsigned int u = __float_as_uint(v);
  const u2 r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__host__ __device__ __forceinline__ int64_t ceil_div(int64_t a, int64_t b) {
  return (a + b - 1) / b;
}

// Index arrays (sequence lengths, start offsets, block tables) arrive as int32 or as int64, as the
// caller's framework holds them; element i is read as the 32-bit word i << sh (sh = 1: the low
// half of a little-endian int64 -- the values are token counts and page numbers below 2^31).
struct IdxArray {
  const int32_t* p;
  int sh;
  __device__ __forceinline__ int operator[](int64_t i) const { return p[i << sh]; }
};
inline IdxArray idx_array(const void* p, int index64_mask, int bit) {
  return IdxArray{(const int32_t*)p, (index64_mask >> bit) & 1};
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// tokens per workgroup of the fused router + chunk-histogram kernel = tokens per alignment chunk
// when the two run as one pipeline: 64 (one pass; twice the workgroups, 8 instead of 12 us for
// the router at 16384 tokens) while that keeps the count table within the 256 rows the fused
// placement kernel reduces, else 128 (two passes)
constexpr int kRouteMaxChunks = 256;
inline int route_chunk_tokens(int64_t T) { return (T + 63) / 64 <= kRouteMaxChunks ? 64 : 128; }
int launch_topk_softmax_count(const void* logits, int logits_dtype, float* weights, int32_t* ids,
                              int64_t T, int E, int K, int64_t ld_logits, int renormalize,
                              int chunk_tokens, int32_t* chunk_counts, hipStream_t s);

// compute units of the device that is current on this thread (256 if it cannot be read), kept
// per device: a process may drive GPUs of different sizes.  The table is filled lazily; two
// threads racing on one entry write the same value.
inline int current_device_cu_count() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> table[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = table[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    table[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// status of the launch just issued on this thread
inline int launch_status() { return hipGetLastError() == hipSuccess ? DLB_OK : DLB_ERR_LAUNCH; }

}  // namespace dlb
