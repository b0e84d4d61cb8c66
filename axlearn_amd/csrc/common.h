// Shared device helpers for the CDNA4 (gfx950) attention kernels: MFMA operand types, LDS address
// casts, bf16 packing and the softmax constants.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

#include "../../include/axl_attn.h"

namespace axl {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short shortx4;
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short shortx8;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int intx4;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned u32x4;

#define AXL_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))

// Running row maxima start at the reference's finite sentinel (axlearn/common/attention_bias.py:43)
// and masked logits are set to -inf: exp2(-inf - finite) is exactly 0, and (finite - finite) never
// produces NaN on rows whose first tiles are fully masked.  (A finite masked value would not do:
// exp2(fma(masked, c, -round(masked * c))) exponentiates the rounding error of a ~1e14 product.)
constexpr float kNegInf = -1e15f;
constexpr float kMasked = -__builtin_inff();
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Exponent offset -lse * log2(e) of the backward kernels (p = exp2(s * c + offset)).  A query row with
// no visible key leaves the forward with lse = -inf (and out = 0); its probabilities are all zero, so
// the offset is a large negative number instead of +inf, which would turn s * c + offset into inf or,
// for a masked s = -inf, NaN.
__device__ __forceinline__ float lse_to_exp2_offset(float lse) {
  return lse == -__builtin_inff() ? -1e30f : lse * -1.4426950408889634f;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ bf16x2 pack_bf16(float a, float b) {
  floatx2 v = {a, b};
  return __builtin_convertvector(v, bf16x2);
}

// Eight fp32 -> one MFMA bf16 operand (round to nearest even, v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16x8 pack_bf16x8(float a0, float a1, float a2, float a3, float a4,
                                              float a5, float a6, float a7) {
  union {
    bf16x8 v;
    bf16x2 p[4];
  } u;
  u.p[0] = pack_bf16(a0, a1);
  u.p[1] = pack_bf16(a2, a3);
  u.p[2] = pack_bf16(a4, a5);
  u.p[3] = pack_bf16(a6, a7);
  return u.v;
}

typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 halfx8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 halfx4;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 halfx2;

// Element type of the 16-bit kernels (template parameter E).  Operands travel through global
// memory, LDS and registers as plain 16-bit patterns in the bf16x2 / bf16x8 / shortx4 carriers
// whatever the type; only the matrix instructions, the rounding of fp32 results to 16 bits and
// the widening of single elements differ.  Both roundings are to nearest even.
struct ElemBf16 {
  static constexpr int kDtype = AXL_BF16;
  static __device__ __forceinline__ floatx16 mfma_32x32x16(bf16x8 a, bf16x8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // The same instruction with its accumulator in VECTOR registers whatever form the compiler picks
  // for the function's other MFMAs (inline assembly; `_zero` starts a chain from 0).  For chains whose
  // result vector ALU code reads: in a kernel compiled with accumulators in AGPRs that saves one
  // v_accvgpr_read per element.  The compiler does not know what the assembly is, so the CALLER keeps
  // the distance the hardware wants between the last MFMA of a chain and the first vector ALU read of
  // its result (12 wait states for this 8-pass MFMA; two later MFMAs in between are enough, the matrix
  // pipe takes them one after the other), and keeps register pressure low enough that the compiler
  // has no reason to copy the accumulator elsewhere right after the chain.  `_last` ends a chain whose
  // result is read right away: the wait states are part of the same statement.
  static __device__ __forceinline__ void mfma_32x32x16_vgpr(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_32x32x16_vgpr_last(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 3" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_32x32x16_vgpr_zero(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ floatx4 mfma_16x16x32(bf16x8 a, bf16x8 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ floatx4 mfma_16x16x16(shortx4 a, shortx4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ bf16x2 pack(float a, float b) { return pack_bf16(a, b); }
  static __device__ __forceinline__ float dot2(bf16x2 a, bf16x2 b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
  }
  static __device__ __forceinline__ float widen(__bf16 bits) { return (float)bits; }
  static __device__ __forceinline__ __bf16 narrow(float x) { return (__bf16)x; }
};
struct ElemF16 {
  static constexpr int kDtype = AXL_F16;
  static __device__ __forceinline__ floatx16 mfma_32x32x16(bf16x8 a, bf16x8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c,
                                                  0, 0, 0);
  }
  static __device__ __forceinline__ void mfma_32x32x16_vgpr(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_32x32x16_vgpr_last(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 3" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_32x32x16_vgpr_zero(bf16x8 a, bf16x8 b, floatx16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ floatx4 mfma_16x16x32(bf16x8 a, bf16x8 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c,
                                                  0, 0, 0);
  }
  static __device__ __forceinline__ floatx4 mfma_16x16x16(shortx4 a, shortx4 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(halfx4, a), __builtin_bit_cast(halfx4, b), c, 0,
                                                 0, 0);
  }
  static __device__ __forceinline__ bf16x2 pack(float a, float b) {
    floatx2 v = {a, b};
    return __builtin_bit_cast(bf16x2, __builtin_convertvector(v, halfx2));
  }
  static __device__ __forceinline__ float dot2(bf16x2 a, bf16x2 b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(halfx2, a), __builtin_bit_cast(halfx2, b), c, false);
  }
  static __device__ __forceinline__ float widen(__bf16 bits) { return (float)__builtin_bit_cast(_Float16, bits); }
  static __device__ __forceinline__ __bf16 narrow(float x) { return __builtin_bit_cast(__bf16, (_Float16)x); }
};

// Tag of the fp32 kernels where a template is shared with the 16-bit ones.
struct ElemF32 {
  static constexpr int kDtype = AXL_F32;
};

// Eight fp32 -> one MFMA operand of element type E.
template <typename E>
__device__ __forceinline__ bf16x8 pack8(float a0, float a1, float a2, float a3, float a4, float a5, float a6,
                                        float a7) {
  union {
    bf16x8 v;
    bf16x2 p[4];
  } u;
  u.p[0] = E::pack(a0, a1);
  u.p[1] = E::pack(a2, a3);
  u.p[2] = E::pack(a4, a5);
  u.p[3] = E::pack(a6, a7);
  return u.v;
}

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane j supplies the
// address of 4 contiguous 16-bit elements; lane i receives, as element e, element (i % 4) of the
// data addressed by lane 4*e + i/4.  With lane j pointing at row (j / 4), columns 4*(j % 4)..+3 of
// a row-major tile, lane i ends up with column i of rows 0..3: a 4x16 -> 16x4 transpose.
__device__ __forceinline__ shortx4 lds_read_tr16(const void* lds_addr) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(AXL_LDS(shortx4, lds_addr));
}

// Exchange with lane ^ 32 through v_permlane32_swap (no LDS round trip): after the swap the two
// results hold, between them, this lane's value and its partner's.
__device__ __forceinline__ float xor32_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Row index permutation that swaps bits 2 and 3.  Feeding MFMA 32x32 A-operand lane m with tile
// row pi(m) makes accumulator register r of lane group g hold tile row 16*(r/8) + 8*g + (r%8), so
// registers 8t..8t+7 are exactly the 8 consecutive rows the next MFMA wants as its K-slice.
__device__ __forceinline__ int swap_bits_2_3(int m) {
  return (m & ~12) | ((m & 4) << 1) | ((m & 8) >> 1);
}

// s_waitcnt vmcnt(0) only (expcnt and lgkmcnt fields left at "no wait").  Placed before a main loop
// it retires the loads of loop-invariant fragments, so the compiler's wait-count bookkeeping does
// not make every iteration wait on the loads it has just issued for the NEXT tile.
__device__ __forceinline__ void wait_all_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// One 16-byte-per-lane direct global->LDS load (global_load_lds_dwordx4): lane l's 16 bytes land at
// lds_base + 16*l, where lds_base is a wave-uniform LDS byte address.  Issued through inline assembly
// so that the compiler neither tracks it nor waits for it; such loads complete in issue order and
// are awaited with wait_vmem_le<N>() (at most N vector-memory operations still outstanding).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16(const void* gsrc, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(lds_base)
               : "memory", "m0");
}
// Two such loads from one scalar base: lane l's two 16-byte pieces come from sbase + voff0 and
// sbase + voff1_biased + 1024 (the instruction offset of the second load moves its global address
// as well as its LDS address, so the caller passes the second offset minus 1024) and land at
// lds_base + 16*l and lds_base + 1024 + 16*l.  No vector instruction forms an address.
__device__ __forceinline__ void dma16x2(unsigned voff0, unsigned voff1_biased, const void* sbase, unsigned lds_base) {
  asm volatile(
      "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024"
      :
      : "v"(voff0), "v"(voff1_biased), "s"(sbase), "s"(lds_base)
      : "memory", "m0");
}
// One such load from a scalar base plus a per-lane byte offset.
__device__ __forceinline__ void dma16s(unsigned voff, const void* sbase, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(sbase), "s"(lds_base)
               : "memory", "m0");
}
// The same for lanes 0..7 only (128 bytes).  The load is issued with EXEC narrowed to those lanes and
// EXEC is then set back to all 64 lanes, so the caller must be in wave-uniform control flow with every
// lane active (no branch is generated, which keeps the caller's code in one scheduling region).
__device__ __forceinline__ void dma16s_first8(unsigned voff, const void* sbase, unsigned lds_base) {
  asm volatile(
      "s_mov_b64 exec, 0xff\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\ts_mov_b64 exec, -1"
      :
      : "v"(voff), "s"(sbase), "s"(lds_base)
      : "memory", "m0");
}
// The same for lanes 0..15 (256 bytes).
__device__ __forceinline__ void dma16s_first16(unsigned voff, const void* sbase, unsigned lds_base) {
  asm volatile(
      "s_mov_b64 exec, 0xffff\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\ts_mov_b64 exec, -1"
      :
      : "v"(voff), "s"(sbase), "s"(lds_base)
      : "memory", "m0");
}
// Two 16-byte-per-lane global stores from one scalar base: lane l's pieces go to sbase + voff and
// sbase + voff + 1024.  Issued through inline assembly like the tile loads, so the compiler's wait
// counts never involve them (vector memory stores count in vmcnt as well).  The data is written once
// and read by a later kernel: streaming policy (write through, no reuse), which costs the issuing
// kernel least (measured against the default and the single-modifier policies).
__device__ __forceinline__ void store16x2(unsigned voff, void* sbase, bf16x8 d0, bf16x8 d1) {
  asm volatile("global_store_dwordx4 %0, %1, %3 sc0 sc1 nt\n\tglobal_store_dwordx4 %0, %2, %3 offset:1024 sc0 sc1 nt"
               :
               : "v"(voff), "v"(d0), "v"(d1), "s"(sbase)
               : "memory");
}
#pragma clang diagnostic pop
template <int N>
__device__ __forceinline__ void wait_vmem_le() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }
// LDS byte address of a pointer into shared memory.
__device__ __forceinline__ unsigned lds_address(const void* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// XOR swizzle of unpadded LDS tiles whose rows hold D bf16 (2D bytes).  Tiles that arrive by direct
// global->LDS loads cannot be padded (an instruction writes 1 KB of consecutive LDS), so bank
// conflicts are avoided by storing the 16-byte chunk c of row R at chunk index c ^ tile_swizzle(R):
// each lane simply fetches the chunk that belongs at its slot.  The map is GF(2)-linear in the
// row's low 4 bits and was found by exhaustive search with a bank simulator: conflict-free for
// row-per-lane 128-bit reads in the row order swap_bits_2_3(lane) and for the transposing 64-bit
// reads (ds_read_b64_tr_b16) alike, under a 32-bank and a 64-bank model.
template <int D>
__device__ __forceinline__ int tile_swizzle(int row) {
  return D == 128 ? (((row & 1) ? 4 : 0) ^ ((row & 2) ? 10 : 0) ^ ((row & 4) ? 1 : 0) ^ ((row & 8) ? 3 : 0))
                  : (((row & 1) ? 2 : 0) ^ ((row & 2) ? 4 : 0) ^ ((row & 4) ? 1 : 0) ^ ((row & 8) ? 3 : 0));
}

// Segment-id pruning of a workgroup's loop range.  `my_id` is the segment id of one of the rows the
// workgroup owns (every owned row is passed by at least one thread); ids[lo, hi) are the segment ids
// of the rows it loops over.  A looped row can only match an owned row if its id lies between the
// smallest and the largest owned id, so [lo, hi) is shrunk to the hull of such rows (empty if there
// is none).  Called by all 256 threads of the workgroup; contains barriers.
__device__ __forceinline__ void shrink_to_segment_hull(int my_id, const int32_t* ids, int tid, int& lo, int& hi) {
  __shared__ int s_rng[4];
  if (tid == 0) {
    s_rng[0] = 0x7fffffff;  // smallest owned id
    s_rng[1] = -0x7fffffff - 1;  // largest owned id
    s_rng[2] = 0x7fffffff;  // first candidate row
    s_rng[3] = -1;          // last candidate row
  }
  __syncthreads();
  atomicMin(&s_rng[0], my_id);
  atomicMax(&s_rng[1], my_id);
  __syncthreads();
  const int id_min = s_rng[0], id_max = s_rng[1];
  int first = 0x7fffffff, last = -1;
  for (int r = lo + tid; r < hi; r += 256) {
    const int id = ids[r];
    if (id >= id_min && id <= id_max) {
      first = min(first, r);
      last = max(last, r);
    }
  }
  if (last >= 0) {
    atomicMin(&s_rng[2], first);
    atomicMax(&s_rng[3], last);
  }
  __syncthreads();
  lo = max(lo, s_rng[2] == 0x7fffffff ? hi : s_rng[2]);
  hi = min(hi, s_rng[3] + 1);
  if (hi < lo) hi = lo;
}

// One pass over the segment ids of the rows [lo, hi) that a workgroup loops over, in groups of GROUP
// consecutive rows (GROUP a multiple of 4; ids 16-byte aligned; the row count a multiple of GROUP):
//   * s_uniform[i], i < cap, gets the id of group g0 + i if its rows all carry one id, else
//     `not_uniform`; g0, the return value, is the first group of the ALIGN-row block that holds row
//     `lo` (ALIGN a multiple of GROUP: the caller's tile size, so that its first tile is covered);
//   * [lo, hi) is shrunk, in whole groups, to the hull of the groups that hold an id between the
//     smallest and the largest id of the workgroup's own rows (`my_id`, passed by every thread): only
//     such a group can hold a row that matches one of them.
// Called by all NT threads of the workgroup; contains barriers.
template <int GROUP, int NT, int ALIGN = GROUP>
__device__ __forceinline__ int classify_segment_groups(int my_id, const int32_t* ids, int tid, int& lo, int& hi,
                                                       int* s_uniform, int cap, int not_uniform) {
  // Reductions go lane to lane inside a wavefront and through one LDS slot per wavefront between
  // them: no atomics (256 threads updating one LDS word take turns).
  __shared__ int s_rng[4 * (NT / 64)];
  const int lane = tid & 63, wave = tid >> 6;
  int id_min = my_id, id_max = my_id;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    id_min = min(id_min, __shfl_xor(id_min, o));
    id_max = max(id_max, __shfl_xor(id_max, o));
  }
  if (lane == 0) {
    s_rng[4 * wave] = id_min;
    s_rng[4 * wave + 1] = id_max;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NT / 64; w++) {
    id_min = min(id_min, s_rng[4 * w]);
    id_max = max(id_max, s_rng[4 * w + 1]);
  }
  // whole ALIGN-row blocks at both ends, so that every group of the caller's first and last tile is described
  const int g0 = (lo / ALIGN) * (ALIGN / GROUP), g1 = ((hi + ALIGN - 1) / ALIGN) * (ALIGN / GROUP);
  int first = 0x7fffffff, last = -1;   // wave-uniform
  for (int base = g0 + wave * 64; base < g1; base += NT) {
    const int i = base + lane;
    bool cand = false;
    if (i < g1) {
      const intx4* p = (const intx4*)(ids + (int64_t)i * GROUP);
      int mn = 0x7fffffff, mx = -0x7fffffff - 1;
#pragma unroll
      for (int v = 0; v < GROUP / 4; v++) {
        const intx4 x = p[v];
        mn = min(min(mn, min(x[0], x[1])), min(x[2], x[3]));
        mx = max(max(mx, max(x[0], x[1])), max(x[2], x[3]));
      }
      if (i - g0 < cap) s_uniform[i - g0] = mn == mx ? mn : not_uniform;
      cand = mx >= id_min && mn <= id_max;
    }
    const uint64_t m = __builtin_amdgcn_ballot_w64(cand);   // lane j looks at group base + j
    if (m) {
      first = min(first, base + (int)__builtin_ctzll(m));
      last = max(last, base + 63 - (int)__builtin_clzll(m));
    }
  }
  if (lane == 0) {
    s_rng[4 * wave + 2] = first;
    s_rng[4 * wave + 3] = last;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NT / 64; w++) {
    first = min(first, s_rng[4 * w + 2]);
    last = max(last, s_rng[4 * w + 3]);
  }
  lo = max(lo, first == 0x7fffffff ? hi : first * GROUP);
  hi = min(hi, (last + 1) * GROUP);
  if (hi < lo) hi = lo;
  // the same in every lane: say so, the callers form scalar addresses from them
  lo = __builtin_amdgcn_readfirstlane(lo);
  hi = __builtin_amdgcn_readfirstlane(hi);
  return __builtin_amdgcn_readfirstlane(g0);
}

// The same classification from a table that one small kernel has filled beforehand (the backward has a
// workspace for it): `tbl` holds, for every group of 32 consecutive rows of this sequence, the
// smallest and the largest segment id in the group.  The workgroup's own rows are the `own_n` groups
// from `own_g0` on, so their id range comes from the table as well: one global load per thread, one
// barrier, no atomics - instead of a pass over the ids themselves whose latencies nothing overlaps
// when a CU holds a single workgroup.  Semantics as classify_segment_groups with GROUP = 32.
// Called by all NT threads of the workgroup (whole wavefronts); contains a barrier.
constexpr int kSegGroupRows = 32;
template <int NT, int ALIGN = kSegGroupRows>
__device__ __forceinline__ int classify_segment_groups_tbl(const int2* tbl, int own_g0, int own_n, int tid, int& lo,
                                                           int& hi, int* s_uniform, int cap, int not_uniform) {
  constexpr int GROUP = kSegGroupRows;
  __shared__ int s_rng[2 * (NT / 64)];
  int id_min = 0x7fffffff, id_max = -0x7fffffff - 1;
  for (int i = 0; i < own_n; i++) {
    const int2 e = tbl[own_g0 + i];
    id_min = min(id_min, e.x);
    id_max = max(id_max, e.y);
  }
  const int g0 = (lo / ALIGN) * (ALIGN / GROUP), g1 = ((hi + ALIGN - 1) / ALIGN) * (ALIGN / GROUP);
  const int lane = tid & 63, wave = tid >> 6;
  int first = 0x7fffffff, last = -1;   // wave-uniform
  for (int base = g0 + wave * 64; base < g1; base += NT) {
    const int i = base + lane;
    bool cand = false;
    if (i < g1) {
      const int2 e = tbl[i];
      if (i - g0 < cap) s_uniform[i - g0] = e.x == e.y ? e.x : not_uniform;
      cand = e.y >= id_min && e.x <= id_max;
    }
    const uint64_t m = __builtin_amdgcn_ballot_w64(cand);   // lane j looks at group base + j
    if (m) {
      first = min(first, base + (int)__builtin_ctzll(m));
      last = max(last, base + 63 - (int)__builtin_clzll(m));
    }
  }
  if (lane == 0) {
    s_rng[2 * wave] = first;
    s_rng[2 * wave + 1] = last;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NT / 64; w++) {
    first = min(first, s_rng[2 * w]);
    last = max(last, s_rng[2 * w + 1]);
  }
  lo = max(lo, first == 0x7fffffff ? hi : first * GROUP);
  hi = min(hi, (last + 1) * GROUP);
  if (hi < lo) hi = lo;
  // the same in every lane: say so, the callers form scalar addresses from them
  lo = __builtin_amdgcn_readfirstlane(lo);
  hi = __builtin_amdgcn_readfirstlane(hi);
  return __builtin_amdgcn_readfirstlane(g0);
}

// Decodes blockIdx.x into (query block, batch, query head).  Workgroup i is dispatched to XCD i % 8.
// When the (batch, kv head) pairs divide evenly over the 8 XCDs, an XCD works through its pairs a
// group at a time: as few pairs as fill its `slots` resident workgroups (one pair when a pair has
// that many query blocks x query heads), heaviest query blocks (most visible keys under a causal
// mask) first across the group.  The workgroups that run together then read the K/V of one or two
// kv heads, which that XCD's L2 holds, and a group still has enough workgroups to keep every CU busy.
__device__ __forceinline__ void decode_block(int bid, int nqb, int B, int Hq, int Hkv, int slots, int& qb,
                                             int& b, int& h) {
  const int G = Hq / Hkv;
  const int npairs = B * Hkv;
  if (npairs % 8 == 0) {
    const int xcd = bid & 7, slot = bid >> 3;
    const int ppx = npairs >> 3;                       // pairs per XCD
    const int per_pair = nqb * G;
    const int pgn = max(1, (slots + per_pair - 1) / per_pair);  // pairs per group
    const int grp = slot / (pgn * per_pair);
    const int r = slot - grp * (pgn * per_pair);
    const int pg = min(pgn, ppx - grp * pgn);          // the last group may be smaller
    const int rem = r % (pg * G);
    const int pair = xcd + 8 * (grp * pgn + rem / G);
    qb = nqb - 1 - r / (pg * G);
    b = pair / Hkv;
    h = (pair % Hkv) * G + rem % G;
  } else {
    const int per_qb = B * Hq;
    const int qb_rev = bid / per_qb, rem = bid % per_qb;
    qb = nqb - 1 - qb_rev;
    b = rem / Hq;
    h = rem % Hq;
  }
}

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}) in order.
template <class F, int... I>
__device__ __forceinline__ void for_each_index_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void for_each_index(F&& f) {
  for_each_index_impl(f, std::make_integer_sequence<int, N>{});
}

// Eight consecutive 16-bit elements of a row, or zeros where the row (of d_real elements, a multiple
// of 8) has already ended: the operand fragments of a head_dim below the compiled width.
__device__ __forceinline__ bf16x8 load8_within(const __bf16* row, int col, int d_real) {
  const bf16x8 zero8 = {};
  return col < d_real ? *(const bf16x8*)(row + col) : zero8;
}

struct Strides3 {
  int64_t b, s, h;
};

// Dense bias / dropout mask of the prefill kernels (AxlAttnAux), in kernel-argument form.
struct AuxArgs {
  const char* bias;     // nullptr = none
  const uint8_t* drop;  // nullptr = none; nonzero byte = dropped
  int64_t bias_sb, bias_sh, bias_sr;  // BYTES per batch / head / query row
  int64_t drop_sb, drop_sh, drop_sr;  // bytes
  int bias_f32;         // element type of bias: 1 fp32, 0 bf16
  float inv_scale;      // 1 / softmax_scale: bias in units of the raw (unscaled) logits
  float keep_scale;     // 1 / (1 - dropout_rate)
};

// Template argument of the kernels that are compiled once per combination of these inputs: which
// of them there are and the element type of the bias (0 = the plain kernel).
constexpr int kAuxBias16 = 1, kAuxBias32 = 2, kAuxDrop = 4;

AuxArgs make_aux_args(const AxlAttnAux& x, float softmax_scale);
int check_aux(const char* who, const AxlAttnAux& x, int batch, int hq, int q_len, int kv_len);

// 4 consecutive bias elements of a row, starting at key `col`, as fp32 (the fp32 kernels' bias read;
// the 16-bit kernels fetch raw words a tile ahead and convert at the use).
template <int N>
__device__ __forceinline__ void load_bias(const char* row, int col, int is_f32, float (&out)[N]) {
  static_assert(N == 4, "four elements per call");
  if (is_f32) {
    const floatx4 v = *(const floatx4*)(row + (int64_t)col * 4);
#pragma unroll
    for (int j = 0; j < 4; j++) out[j] = v[j];
  } else {
    union {
      uint32_t u[2];
      __bf16 e[4];
    } w;
    const uint2 v = *(const uint2*)(row + (int64_t)col * 2);
    w.u[0] = v.x; w.u[1] = v.y;
#pragma unroll
    for (int i = 0; i < 4; i++) out[i] = (float)w.e[i];
  }
}

// ---- fp32 products on the 16-bit matrix instruction (the fp32 kernels).  An fp32 operand travels as three
// bf16 values, x = hi + mid + lo, each the rounded remainder of the one before (8 + 8 + 8 bits of
// significand: the split is exact); a product is formed from the six partial products that matter and
// accumulated in fp32 by the instruction.
// Two fp32 values as three pairs of bf16: hi = rn(x), mid = rn(x - hi), lo = rn(x - hi - mid).
struct Split3x2 {
  bf16x2 part[3];
};
__device__ __forceinline__ Split3x2 split3(float x0, float x1) {
  Split3x2 r;
  r.part[0] = pack_bf16(x0, x1);
  const unsigned hb = __builtin_bit_cast(unsigned, r.part[0]);
  const float r0 = x0 - __uint_as_float(hb << 16), r1 = x1 - __uint_as_float(hb & 0xffff0000u);
  r.part[1] = pack_bf16(r0, r1);
  const unsigned mb = __builtin_bit_cast(unsigned, r.part[1]);
  r.part[2] = pack_bf16(r0 - __uint_as_float(mb << 16), r1 - __uint_as_float(mb & 0xffff0000u));
  return r;
}
// Eight fp32 values as the three MFMA operands hi, mid, lo.
struct Split3x8 {
  union {
    bf16x8 v;
    bf16x2 p[4];
  } part[3];
};
__device__ __forceinline__ void split3x8(const float (&x)[8], Split3x8& out) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const Split3x2 s = split3(x[2 * i], x[2 * i + 1]);
#pragma unroll
    for (int p = 0; p < 3; p++) out.part[p].p[i] = s.part[p];
  }
}
// c += a b from the split operands: the six partial products, the small ones first.
__device__ __forceinline__ floatx16 mfma_split(const bf16x8 (&a)[3], const bf16x8 (&b)[3], floatx16 c) {
  c = ElemBf16::mfma_32x32x16(a[2], b[0], c);
  c = ElemBf16::mfma_32x32x16(a[0], b[2], c);
  c = ElemBf16::mfma_32x32x16(a[1], b[1], c);
  c = ElemBf16::mfma_32x32x16(a[1], b[0], c);
  c = ElemBf16::mfma_32x32x16(a[0], b[1], c);
  c = ElemBf16::mfma_32x32x16(a[0], b[0], c);
  return c;
}

int set_error(int code, const char* fmt, ...);

// Raises a kernel's dynamic LDS limit to `bytes` (hipFuncAttributeMaxDynamicSharedMemorySize) the
// first time the kernel is launched on the current device; later launches only look the pair up.
hipError_t allow_dynamic_lds(const void* kernel, int bytes);

// Compute units of the current device, looked up once (defined in api.hip).
int cu_count();

}  // namespace axl
