// Pieces shared by the attention kernels: element traits and the argument block.
#pragma once
#include "common.h"

namespace bsa {

constexpr float kLog2e = 1.4426950408889634f;

struct AttnBf16 {
  using elem_t = uint16_t;
  __device__ static float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
  __device__ static uint16_t round(float v) {
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
};

struct AttnF16 {
  using elem_t = uint16_t;
  __device__ static float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
  __device__ static uint16_t round(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};

struct AttnF32 {
  using elem_t = float;
  __device__ static float widen(float v) { return v; }
  __device__ static float round(float v) { return v; }
};

// value of a mask element (any non-zero value masks the position)
__device__ inline bool mask_set(const void *mask, int kind, int64_t idx) {
  if (kind == 1) return static_cast<const uint8_t *>(mask)[idx] != 0;
  return false;
}

// One entry of a grouped forward list, 64 bytes (BSA_ATTN_RECORD_INTS int32): the list entry (key block in
// the low 28 bits, bit 28 + g set if the key block is active for query block g of the group), the packed
// indices of its K and V head slices (-1: inactive or no such slice) and of its mask and bias blocks for
// either query block of the group (-1: none).
struct AttnFwdRecord {
  int32_t entry, pk[2], pv[2], pm[2], pb[2], pad[7];
};
static_assert(sizeof(AttnFwdRecord) == BSA_ATTN_RECORD_INTS * 4, "record layout");

int attn_fwd_generic(const bsa_attn_args &a, hipStream_t s);
int attn_fwd_records(const bsa_attn_args &a, const int32_t *entries, int32_t *records, hipStream_t s);
int attn_bwd_generic(const bsa_attn_args &a, hipStream_t s);
// MFMA paths; return 1 if the configuration is not covered (caller falls back to the generic kernels)
int attn_fwd_mfma(const bsa_attn_args &a, hipStream_t s);
int attn_fwd_f32mma(const bsa_attn_args &a, hipStream_t s);
int attn_bwd_f32mma(const bsa_attn_args &a, hipStream_t s);
int attn_bwd_mfma(const bsa_attn_args &a, hipStream_t s);
int attn_mask_dead(const void *mask, int64_t n_mask_blocks, uint8_t *dead, hipStream_t s);
size_t attn_bwd_scratch_bytes(int64_t B, int64_t nq, int64_t nk, int64_t n_layout_blocks, int64_t n_mask_blocks);
size_t attn_bwd_ds_bytes(int64_t n_layout_blocks);

}  // namespace bsa
