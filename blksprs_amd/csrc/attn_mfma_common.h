// Pieces shared by the matrix-core attention kernels (forward and backward): operand traits, LDS layouts of
// 64 x 64 16-bit tiles, the asynchronous global -> LDS copy.
#pragma once
#include "attn_common.h"

namespace bsa {
namespace mfma {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct MBf16 {
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
  // a.lo * b.lo + a.hi * b.hi + c for two packed pairs of elements, in fp32: one instruction
  __device__ static float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  }
};

struct MF16 {
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
  __device__ static float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  }
};

constexpr int kSbs = 64;
constexpr int kBlockBytes = kSbs * kSbs * 2;  // one 16-bit block

// XOR applied to the 16-byte chunk index of row r of a tile that is read both ways: by rows (128-bit reads
// serve 8 lanes = 8 consecutive rows at a time, one chunk each: they need eight different values) and with
// the transposing LDS load (it serves 32 lanes at a time = four rows r .. r + 3, r a multiple of 4, 64
// consecutive bytes of each; two 128-byte rows span the 64 banks once, so rows r and r + 2 must put their 64
// bytes into different halves of the row: bit 2 of the value is bit 1 of the row).  Depends on r % 8 only.
__device__ static inline int t_swizzle(int r) { return (((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1) | (r & 1); }

typedef short i16x4 __attribute__((ext_vector_type(4)));

// Operand fragment whose eight contraction indices run over the ROWS of a row-major 64 x 64 16-bit tile
// (chunks swizzled with t_swizzle): lane l gets column col0 + l % 16 of rows row0 .. + 3 and row0 + 8 .. + 11,
// where col0 and row0 may differ between the four 16-lane groups.  The transposing load gives lane i of a
// group element t = tile[row0 + t][col0 + i] when lane s of the group points at tile[row0 + s / 4][col0 + 4 (s % 4)].
__device__ static inline u32x4 frag_cols_t(const char *lds, int row0, int col0, int lane) {
  const int s = lane & 15;
  const int r = row0 + (s >> 2), c = col0 + 4 * (s & 3);
  const char *p0 = lds + r * 128 + ((((c >> 3) ^ t_swizzle(r))) << 4) + ((c & 4) << 1);
  const int r8 = r + 8;
  const char *p1 = lds + r8 * 128 + ((((c >> 3) ^ t_swizzle(r8))) << 4) + ((c & 4) << 1);
  const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)p0);
  const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)p1);
  const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
  return u32x4{l2[0], l2[1], h2[0], h2[1]};
}

// The values of lanes l and l ^ 32 of a wave, combined: one v_permlane32_swap (lanes 32 .. 63 of the first operand
// trade places with lanes 0 .. 31 of the second; with the same value in both, one result holds the lower half's
// values in both halves and the other the upper half's), no trip through LDS as a shuffle takes.  Every lane gets
// lower (op) upper, so for a sum both lanes of a pair hold the same bits.
__device__ static inline float max_across32(float v) {
  float lower = v, upper = v;  // spelled out: two registers that hold the same value, both read and written
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
  return fmaxf(lower, upper);
}
__device__ static inline float sum_across32(float v) {
  float lower = v, upper = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
  return lower + upper;
}

__device__ static inline int first_lane(int v) { return __builtin_amdgcn_readfirstlane(v); }
typedef __attribute__((address_space(3))) void *lds_ptr_t;

// Asynchronous copy of 64 x 16 bytes, global -> LDS: lane l's 16 bytes land at dst + 16 l (dst is wave
// uniform).  Completion is counted by vmcnt like any vector load.  Written as inline assembly so that the
// compiler's wait-count pass does not see it: it would otherwise wait for the copy in front of every later
// LDS read, also reads of other LDS arrays.  m0 is a reserved register for clang's AMDGPU backend (it is never allocated
// to a value that lives across statements: the backend writes it immediately in front of each of its own uses,
// and naming it in a clobber list is diagnosed as undefined behaviour), so overwriting it here is safe.  The caller waits (vmcnt(0)) before the data is read.  Copies
// the compiler does not know about only make the waits it computes for its own loads longer, never shorter.
// The source is base (wave uniform) + off (per lane, 32 bits).
__device__ static inline void copy_1k_to_lds(const char *base, uint32_t off, char *dst) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr_t)dst;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(off), "s"(base), "s"(lds_addr)
               : "memory");
}

// Two such copies with one address setup: the KiB at base + off and the KiB 1024 bytes further on, to dst and
// dst + 1024 (the instruction's offset field moves both the global and the LDS address).
__device__ static inline void copy_2k_to_lds(const char *base, uint32_t off, char *dst) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr_t)dst;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024"
               :
               : "v"(off), "s"(base), "s"(lds_addr)
               : "memory");
}

// 16 bytes at base (wave uniform) + off (per lane): scalar base, 32-bit vector offset addressing
__device__ static inline u32x4 load16(const char *base, uint32_t off) {
  return *reinterpret_cast<const u32x4 *>(base + off);
}

}  // namespace mfma
}  // namespace bsa
