// hipDMA memory primitives: fixed-size register chunks and the loads/stores
// that fill and drain them.  Plays the role of the PTX ld/st wrappers of
// include/cudaDMAv2.h:80-679 and of the register buffers of
// include/cudaDMAv2.h:686-1310, for gfx950:
//   * a chunk is ALIGNMENT bytes (4, 8 or 16) = 1, 2 or 4 VGPRs and is moved by
//     global_load_dword/x2/x4 (source known global), flat_load_* (generic
//     source), ds_write_b32/b64/b128 (destination known LDS) or a generic store;
//   * a ragged tail of 4, 8 or 12 bytes is moved in dword pieces;
//   * the direct path uses global_load_lds_dwordx4 / _dword, which writes
//     M0-base + lane*size in LDS without touching a VGPR.
#pragma once

#include "base.hpp"

namespace hipdma {
namespace detail {

typedef unsigned u32x1_t;
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

template<int BYTES> struct chunk_of;
template<> struct chunk_of<4>  { typedef u32x1_t type; };
template<> struct chunk_of<8>  { typedef u32x2_t type; };
template<> struct chunk_of<16> { typedef u32x4_t type; };

#define HIPDMA_GLOBAL_AS __attribute__((address_space(1)))
#define HIPDMA_LDS_AS    __attribute__((address_space(3)))

// Cache-policy bits of a gfx950 vector memory instruction (the `aux` operand of the direct-to-LDS
// loads: 1 = sc0, 2 = nt, 16 = sc1) for each load qualifier of include/cudaDMAv2.h:50-56:
//   LOAD_CACHE_ALL       (ld.ca)  none: cached in the vector L1 and in L2
//   LOAD_CACHE_GLOBAL    (ld.cg)  sc1: device scope, the vector L1 is bypassed and L2 serves the load
//   LOAD_CACHE_STREAMING (ld.cs)  nt: non-temporal, the line is first in line for eviction
//   LOAD_CACHE_LAST_USE  (ld.lu)  nt: the closest policy there is
//   LOAD_CACHE_VOLATILE  (ld.cv)  sc0 sc1: system scope, fetched again on every access
__host__ __device__ constexpr int load_policy_bits(const int q)
{
  return (q == LOAD_CACHE_STREAMING || q == LOAD_CACHE_LAST_USE) ? 2
       : (q == LOAD_CACHE_VOLATILE) ? 17
       : (q == LOAD_CACHE_GLOBAL) ? 16 : 0;
}

// One aligned vector load of sizeof(T) bytes, P = pointer type in the address space of the source.
// The compiler offers sc1 alone only through an agent-scope atomic load, which exists for 4 and 8
// bytes: a 16-byte LOAD_CACHE_GLOBAL load is issued as two dwordx2 loads with sc1.  (One dwordx4 with
// sc0 sc1 would bypass the vector L1 as well, but system-scope loads have a much longer latency: a
// read-only stream of 1 GiB ran at 2.4 TB/s with them at one workgroup per compute unit, at 6.0 TB/s
// with the two sc1 halves, 6.3 TB/s plain and 6.4 TB/s non-temporal.)
template<typename T, int LOAD_QUAL, typename P>
__device__ __forceinline__ T load_vec_from(P p)
{
  if constexpr (LOAD_QUAL == LOAD_CACHE_STREAMING || LOAD_QUAL == LOAD_CACHE_LAST_USE) {
    return __builtin_nontemporal_load(p);
  } else if constexpr (LOAD_QUAL == LOAD_CACHE_VOLATILE) {
    return *(volatile typename std::remove_pointer<P>::type*)p;     // volatile added, address space kept
  } else if constexpr (LOAD_QUAL == LOAD_CACHE_GLOBAL && sizeof(T) == 16) {
    const unsigned long long* q = (const unsigned long long*)p;
    const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    T out;
    out[0] = (unsigned)lo;
    out[1] = (unsigned)(lo >> 32);
    out[2] = (unsigned)hi;
    out[3] = (unsigned)(hi >> 32);
    return out;
  } else if constexpr (LOAD_QUAL == LOAD_CACHE_GLOBAL && sizeof(T) == 4) {
    return (T)__hip_atomic_load((const unsigned*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if constexpr (LOAD_QUAL == LOAD_CACHE_GLOBAL && sizeof(T) == 8) {
    const unsigned long long v = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    T out;
    out[0] = (unsigned)v;
    out[1] = (unsigned)(v >> 32);
    return out;
  } else {
    return *p;
  }
}

template<typename T, bool GLOBAL_LOAD, int LOAD_QUAL>
__device__ __forceinline__ T load_vec(const void* ptr)
{
  if constexpr (GLOBAL_LOAD) return load_vec_from<T, LOAD_QUAL>((const HIPDMA_GLOBAL_AS T*)ptr);
  else return load_vec_from<T, LOAD_QUAL>((const T*)ptr);
}

// One aligned vector store of sizeof(T) bytes.  The reference's stores take generic addresses
// (include/cudaDMAv2.h:553-679); so do these, except for the STORE_LDS* additions.
//   STORE_WRITE_BACK          (st.wb)  plain store
//   STORE_CACHE_GLOBAL        (st.cg)  plain store: the vector L1 is write-through and does not allocate on a
//                                      store, so every store is already held in L2 only
//   STORE_CACHE_STREAMING     (st.cs)  nt
//   STORE_CACHE_WRITE_THROUGH (st.wt)  sc0 sc1: system scope, written through L2
template<typename T, int STORE_QUAL>
__device__ __forceinline__ void store_vec(const T& value, void* ptr)
{
  if constexpr (store_is_lds(STORE_QUAL)) {
    *(HIPDMA_LDS_AS T*)ptr = value;
  } else if constexpr (STORE_QUAL == STORE_CACHE_STREAMING) {
    __builtin_nontemporal_store(value, (T*)ptr);
  } else if constexpr (STORE_QUAL == STORE_CACHE_WRITE_THROUGH) {
    *(volatile T*)ptr = value;
  } else {
    *(T*)ptr = value;
  }
}

// Word i of a chunk (i is a compile-time constant after unrolling).
template<typename C>
__device__ __forceinline__ unsigned get_word(const C& c, const int i)
{
  if constexpr (std::is_same<C, u32x1_t>::value) return c; else return c[i];
}
template<typename C>
__device__ __forceinline__ void set_word(C& c, const int i, const unsigned v)
{
  if constexpr (std::is_same<C, u32x1_t>::value) c = v; else c[i] = v;
}

// Fill the first `nbytes` (a multiple of 4, 0 < nbytes <= CHUNK) of a CHUNK-byte
// register chunk from an address that is only guaranteed PIECE-byte aligned.
// PIECE == CHUNK and nbytes == CHUNK is the single-instruction fast path.
template<int CHUNK, int PIECE, bool GLOBAL_LOAD, int LOAD_QUAL>
__device__ __forceinline__ void load_chunk(typename chunk_of<CHUNK>::type& c, const char* ptr, const int nbytes)
{
  typedef typename chunk_of<CHUNK>::type chunk_t;
  if constexpr (PIECE == CHUNK) {
    if (nbytes == CHUNK) {
      c = load_vec<chunk_t, GLOBAL_LOAD, LOAD_QUAL>(ptr);
      return;
    }
  }
  typedef typename chunk_of<PIECE>::type piece_t;
  constexpr int WORDS_PER_PIECE = PIECE / 4;
#pragma unroll
  for (int p = 0; p < CHUNK / PIECE; ++p) {
    const int rem = nbytes - p * PIECE;
    if (rem >= PIECE) {
      const piece_t v = load_vec<piece_t, GLOBAL_LOAD, LOAD_QUAL>(ptr + p * PIECE);
#pragma unroll
      for (int w = 0; w < WORDS_PER_PIECE; ++w)
        set_word(c, p * WORDS_PER_PIECE + w, get_word(v, w));
    } else {
#pragma unroll
      for (int w = 0; w < WORDS_PER_PIECE; ++w)
        if (rem > 4 * w)
          set_word(c, p * WORDS_PER_PIECE + w,
                   load_vec<u32x1_t, GLOBAL_LOAD, LOAD_QUAL>(ptr + p * PIECE + 4 * w));
    }
  }
}

template<int CHUNK, int PIECE, int STORE_QUAL>
__device__ __forceinline__ void store_chunk(const typename chunk_of<CHUNK>::type& c, char* ptr, const int nbytes)
{
  typedef typename chunk_of<CHUNK>::type chunk_t;
  if constexpr (PIECE == CHUNK) {
    if (nbytes == CHUNK) {
      store_vec<chunk_t, STORE_QUAL>(c, ptr);
      return;
    }
  }
  typedef typename chunk_of<PIECE>::type piece_t;
  constexpr int WORDS_PER_PIECE = PIECE / 4;
#pragma unroll
  for (int p = 0; p < CHUNK / PIECE; ++p) {
    const int rem = nbytes - p * PIECE;
    if (rem >= PIECE) {
      piece_t v;
#pragma unroll
      for (int w = 0; w < WORDS_PER_PIECE; ++w)
        set_word(v, w, get_word(c, p * WORDS_PER_PIECE + w));
      store_vec<piece_t, STORE_QUAL>(v, ptr + p * PIECE);
    } else {
#pragma unroll
      for (int w = 0; w < WORDS_PER_PIECE; ++w)
        if (rem > 4 * w)
          store_vec<u32x1_t, STORE_QUAL>(get_word(c, p * WORDS_PER_PIECE + w), ptr + p * PIECE + 4 * w);
    }
  }
}

// Direct global -> LDS move of BYTES (4 or 16) per active lane.  `lds_wave_base`
// must be the same for every lane of the wavefront; lane L lands at
// lds_wave_base + L*BYTES.
template<int BYTES, int LOAD_QUAL = LOAD_CACHE_ALL>
__device__ __forceinline__ void load_to_lds(const char* global_lane_ptr, char* lds_wave_base)
{
  static_assert(BYTES == 4 || BYTES == 16, "global_load_lds moves 4 or 16 bytes per lane here");
  // the size and the cache-policy operands have to be literals
  if constexpr (BYTES == 16)
    __builtin_amdgcn_global_load_lds((const HIPDMA_GLOBAL_AS void*)global_lane_ptr,
                                     (HIPDMA_LDS_AS void*)lds_wave_base, 16, 0, load_policy_bits(LOAD_QUAL));
  else
    __builtin_amdgcn_global_load_lds((const HIPDMA_GLOBAL_AS void*)global_lane_ptr,
                                     (HIPDMA_LDS_AS void*)lds_wave_base, 4, 0, load_policy_bits(LOAD_QUAL));
}

// The same move with the source address split into a part that is the same in every lane, held
// in scalar registers, and a 32-bit offset per lane: no vector ALU instruction is needed to form
// the address.  Written as assembly because the compiler only picks this form of the instruction
// when it finds the zero-extension of the lane offset in the same basic block as the load, and it
// moves a loop-invariant one out of the loop.  It does not count the load among the LDS writes it
// tracks: the caller waits with wait_lds_direct() / wait_lds_direct_but<N>(), as for load_to_lds().
// `scalar_base` and `lds_wave_base` must come out of scalar_u32() / scalar_ptr() or scalar
// arithmetic on such values.
__device__ __forceinline__ unsigned scalar_u32(const unsigned v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const char* scalar_ptr(const char* p)
{
  const unsigned long long bits = (unsigned long long)p;
  return (const char*)(((unsigned long long)scalar_u32((unsigned)(bits >> 32)) << 32) | (unsigned long long)scalar_u32((unsigned)bits));
}
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"      // m0 is a reserved register: naming it keeps the compiler from merging its own writes across this one
#define HIPDMA_LOAD_TO_LDS_ASM(INSN, POLICY)                                                  \
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\t" INSN " %0, %1" POLICY                          \
               : : "v"(lane_offset), "s"(scalar_base), "s"(lds_wave_base) : "memory", "m0")
template<int BYTES, int LOAD_QUAL = LOAD_CACHE_ALL>
__device__ __forceinline__ void load_to_lds_scalar_base(const char* scalar_base, const unsigned lane_offset,
                                                        const unsigned lds_wave_base)
{
  static_assert(BYTES == 4 || BYTES == 16, "global_load_lds moves 4 or 16 bytes per lane here");
  constexpr int bits = load_policy_bits(LOAD_QUAL);
  if constexpr (BYTES == 16) {
    if constexpr (bits == 2) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dwordx4", " nt");
    else if constexpr (bits == 16) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dwordx4", " sc1");
    else if constexpr (bits == 17) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dwordx4", " sc0 sc1");
    else HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dwordx4", "");
  } else {
    if constexpr (bits == 2) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dword", " nt");
    else if constexpr (bits == 16) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dword", " sc1");
    else if constexpr (bits == 17) HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dword", " sc0 sc1");
    else HIPDMA_LOAD_TO_LDS_ASM("global_load_lds_dword", "");
  }
}
#undef HIPDMA_LOAD_TO_LDS_ASM
#pragma clang diagnostic pop

// Wait until every global -> LDS move of this wavefront has landed.
__device__ __forceinline__ void wait_lds_direct()
{
  // s_waitcnt vmcnt(0): simm16 = vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]
  __builtin_amdgcn_s_waitcnt(0x0F70);
}

// Wait until all but the YOUNGER most recent vector-memory operations of this wavefront have
// completed (they complete in issue order).
template<int YOUNGER>
__device__ __forceinline__ void wait_lds_direct_but()
{
  static_assert(YOUNGER >= 0 && YOUNGER < 64, "vmcnt holds six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (YOUNGER & 15) | ((YOUNGER >> 4) << 14));
}

// Lane number inside the wavefront.
__device__ __forceinline__ int lane_id()
{
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

}  // namespace detail
}  // namespace hipdma
