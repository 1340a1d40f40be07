// C ABI of block-sparse flash attention: argument checks and the choice between the 16-bit matrix-core kernels
// (16-bit operands, 64 x 64 blocks, at most two head slices), the fp32 matrix-core kernels (every other operand
// type and block size) and the generic kernels (what neither takes: more head slices than fit LDS).
#include "attn_common.h"

namespace {

int check_args(const char *who, const bsa_attn_args *a, bool backward) {
  BSA_REQUIRE(a != nullptr, "%s: NULL argument block", who);
  BSA_REQUIRE(a->sbs == 16 || a->sbs == 32 || a->sbs == 64, "%s: sbs must be 16, 32 or 64 (got %d)", who, a->sbs);
  BSA_REQUIRE(a->dtype == BSA_F32 || a->dtype == BSA_F16 || a->dtype == BSA_BF16, "%s: unknown dtype %d", who,
              a->dtype);
  BSA_REQUIRE(a->B >= 0 && a->nq >= 0 && a->nk >= 0 && a->nh >= 0 && a->nhv >= 0, "%s: negative layout size", who);
  BSA_REQUIRE(a->n_q_blocks >= 0 && a->n_k_blocks >= 0 && a->n_v_blocks >= 0 && a->n_o_blocks >= 0 &&
                  a->n_mask_blocks >= 0 && a->n_bias_blocks >= 0,
              "%s: negative block count", who);
  BSA_REQUIRE(a->mask_kind == 0 || a->mask_kind == 1, "%s: mask_kind must be 0 or 1", who);
  BSA_REQUIRE((a->mask != nullptr) == (a->mask_kind == 1), "%s: mask pointer and mask_kind disagree", who);
  if (a->B * a->nq == 0 && a->B * a->nk == 0) return BSA_OK;
  BSA_REQUIRE(a->key_offsets != nullptr, "%s: key_offsets is NULL", who);
  BSA_REQUIRE(a->lse != nullptr || a->B * a->nq == 0, "%s: lse is NULL", who);
  BSA_REQUIRE(a->nh == 0 || (a->pidx_q && a->pidx_k), "%s: pidx_q / pidx_k is NULL", who);
  BSA_REQUIRE(a->nhv == 0 || (a->pidx_v && a->pidx_o), "%s: pidx_v / pidx_o is NULL", who);
  BSA_REQUIRE(!a->mask || a->pidx_mask, "%s: mask without pidx_mask", who);
  BSA_REQUIRE(!a->bias || a->pidx_bias, "%s: bias without pidx_bias", who);
  BSA_REQUIRE(a->B * a->nq < 0x7fffffffLL && a->B * a->nk < 0x7fffffffLL, "%s: too many sequence blocks", who);
  BSA_REQUIRE(a->nh < 65536 && a->nhv < 65536, "%s: too many head slices", who);
  BSA_REQUIRE(a->group_size >= 0 && a->group_size <= 2, "%s: group_size must be 0, 1 or 2", who);
  BSA_REQUIRE(a->group_size == 0 || a->group_offsets, "%s: group_size without group_offsets", who);
  if (backward) {
    BSA_REQUIRE(a->query_offsets != nullptr, "%s: query_offsets is NULL", who);
    BSA_REQUIRE(a->delta != nullptr || a->B * a->nq == 0, "%s: delta is NULL", who);
    BSA_REQUIRE(a->n_o_blocks == 0 || (a->o && a->d_o), "%s: o / d_o is NULL", who);
    BSA_REQUIRE(a->n_q_blocks == 0 || a->dq, "%s: dq is NULL", who);
    BSA_REQUIRE(a->n_k_blocks == 0 || a->dk, "%s: dk is NULL", who);
    BSA_REQUIRE(a->n_v_blocks == 0 || a->dv, "%s: dv is NULL", who);
    BSA_REQUIRE(!a->dbias || a->bias, "%s: dbias without bias", who);
  } else {
    BSA_REQUIRE(a->n_o_blocks == 0 || a->o, "%s: o is NULL", who);
  }
  return BSA_OK;
}

}  // namespace

extern "C" int bsa_attn_fwd(const bsa_attn_args *args, bsa_stream_t stream) {
  if (int rc = check_args("bsa_attn_fwd", args, false)) return rc;
  hipStream_t s = bsa::as_stream(stream);
  int rc = bsa::attn_fwd_mfma(*args, s);          // 16-bit operands, 64 x 64 blocks
  if (rc == 1) rc = bsa::attn_fwd_f32mma(*args, s);  // everything else, on the fp32 matrix-core instruction
  if (rc == 1) rc = bsa::attn_fwd_generic(*args, s);
  return rc;
}

extern "C" int bsa_attn_fwd_records(const bsa_attn_args *a, const int32_t *group_entries, int32_t *records,
                                    bsa_stream_t stream) {
  const char *who = "bsa_attn_fwd_records";
  BSA_REQUIRE(a != nullptr, "%s: NULL argument block", who);
  BSA_REQUIRE(a->group_size == 1 || a->group_size == 2, "%s: group_size must be 1 or 2 (got %d)", who, a->group_size);
  BSA_REQUIRE(a->B >= 0 && a->nq >= 0 && a->nk >= 0, "%s: negative layout size", who);
  BSA_REQUIRE(a->nh >= 0 && a->nh <= 2 && a->nhv >= 0 && a->nhv <= 2, "%s: at most two head slices", who);
  BSA_REQUIRE(a->nk < (1 << 28), "%s: too many key blocks for a list entry", who);
  if (a->B * a->nq == 0) return BSA_OK;
  BSA_REQUIRE(a->group_offsets != nullptr, "%s: group_offsets is NULL", who);
  BSA_REQUIRE(a->nh == 0 || a->pidx_k, "%s: pidx_k is NULL", who);
  BSA_REQUIRE(a->nhv == 0 || a->pidx_v, "%s: pidx_v is NULL", who);
  BSA_REQUIRE(a->B * ((a->nq + a->group_size - 1) / a->group_size) < 0x7fffffffLL, "%s: too many groups", who);
  if (group_entries == nullptr || records == nullptr) return BSA_OK;  // no entries
  return bsa::attn_fwd_records(*a, group_entries, records, bsa::as_stream(stream));
}

extern "C" int bsa_attn_mask_dead(const void *mask, int64_t n_mask_blocks, int32_t sbs, uint8_t *dead,
                                  bsa_stream_t stream) {
  const char *who = "bsa_attn_mask_dead";
  BSA_REQUIRE(sbs == 64, "%s: only 64 x 64 blocks (got %d)", who, sbs);
  BSA_REQUIRE(n_mask_blocks >= 0 && n_mask_blocks < 0x7fffffffLL, "%s: bad number of mask blocks", who);
  if (n_mask_blocks == 0) return BSA_OK;
  BSA_REQUIRE(mask != nullptr && dead != nullptr, "%s: NULL argument", who);
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(mask) & 15) == 0, "%s: mask must be 16-byte aligned", who);
  return bsa::attn_mask_dead(mask, n_mask_blocks, dead, bsa::as_stream(stream));
}

extern "C" size_t bsa_attn_bwd_scratch_bytes(int64_t B, int64_t nq, int64_t nk, int64_t n_layout_blocks,
                                             int64_t n_mask_blocks) {
  if (B < 0 || nq < 0 || nk < 0 || n_layout_blocks < 0 || n_mask_blocks < 0) return 0;
  return bsa::attn_bwd_scratch_bytes(B, nq, nk, n_layout_blocks, n_mask_blocks);
}

extern "C" size_t bsa_attn_bwd_ds_bytes(int64_t n_layout_blocks, int32_t sbs) {
  if (n_layout_blocks < 0 || sbs != 64) return 0;
  return bsa::attn_bwd_ds_bytes(n_layout_blocks);
}

extern "C" int bsa_attn_bwd(const bsa_attn_args *args, bsa_stream_t stream) {
  if (int rc = check_args("bsa_attn_bwd", args, true)) return rc;
  BSA_REQUIRE(args->bwd_scratch == nullptr || args->n_layout_blocks >= 0, "bsa_attn_bwd: negative n_layout_blocks");
  BSA_REQUIRE(args->bwd_scratch_bytes >= 0, "bsa_attn_bwd: negative bwd_scratch_bytes");
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(args->bwd_scratch) & 15) == 0, "bsa_attn_bwd: bwd_scratch must be 16-byte aligned");
  BSA_REQUIRE(args->bwd_ds_bytes >= 0, "bsa_attn_bwd: negative bwd_ds_bytes");
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(args->bwd_ds) & 15) == 0, "bsa_attn_bwd: bwd_ds must be 16-byte aligned");
  if (args->bwd_scratch != nullptr && args->bwd_scratch_bytes > 0) {
    const size_t need = bsa::attn_bwd_scratch_bytes(args->B, args->nq, args->nk, args->n_layout_blocks, args->n_mask_blocks);
    BSA_REQUIRE((size_t)args->bwd_scratch_bytes >= need, "bsa_attn_bwd: bwd_scratch holds %lld bytes, %zu are needed",
                (long long)args->bwd_scratch_bytes, need);
  }
  hipStream_t s = bsa::as_stream(stream);
  int rc = bsa::attn_bwd_mfma(*args, s);
  if (rc == 1) rc = bsa::attn_bwd_f32mma(*args, s);
  if (rc == 1) rc = bsa::attn_bwd_generic(*args, s);
  return rc;
}
