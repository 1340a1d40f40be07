// Row-wise softmax over the active blocks of a block row (fp32), forward and backward.
//
// The blocks of one block row are consecutive in the compressed tensor (row-major
// block order), so a row is `count` whole blocks starting at row_offsets[r].  One
// wavefront owns a group of element rows of one block row and reads them with one
// float4 per lane: for sbs <= 256 the 64 lanes cover 256 consecutive floats of a
// block (256/sbs element rows), so every wave load is one contiguous KiB.  The max /
// sum reductions stay inside the sbs/4 lanes of an element row (xor shuffles).
// Rows of up to 32 float4 units per lane stay in registers between the reduction
// and the write (one HBM read + one write); longer rows make two read passes.
#include "common.h"

namespace {

constexpr int kMaxUnits = 32;
constexpr int kWaves = 4;  // waves (tasks) per workgroup

struct RowGeom {
  int sbs_log2;
  int lpr;       // lanes per element row = min(64, sbs/4)
  int nq_log2;   // float4 units per lane per block = max(1, sbs/256), as log2
  int groups_log2;  // wave tasks per block row = sbs * lpr / 64, as log2
};

// The reductions over the lpr lanes of an element row, without a trip through LDS (a shuffle computes a lane
// address, goes through LDS and waits for it).  Steps 1 and 2 exchange inside a group of four lanes (DPP quad_perm);
// after them the four lanes of a group agree, so mirroring a half row (lane i <-> 7 - i) pairs every group with its
// neighbour and mirroring a row (i <-> 15 - i) pairs the two halves of 16 lanes: partners other than those of an
// xor exchange, holding the same values.  Steps 16 and 32 trade register halves (v_permlane16_swap /
// v_permlane32_swap with the same value in both operands: one result holds the even groups' values twice, the other
// the odd groups').  Every step combines a value with its partner's by a commutative operation, so all lanes of a
// row end with the same bits, as with xor shuffles.
template <int CTRL>
__device__ inline float dpp_partner(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <typename Op>
__device__ inline float lanes_reduce(float v, int lpr, Op op) {
  if (lpr > 1) v = op(v, dpp_partner<0xB1>(v));   // quad_perm [1, 0, 3, 2]
  if (lpr > 2) v = op(v, dpp_partner<0x4E>(v));   // quad_perm [2, 3, 0, 1]
  if (lpr > 4) v = op(v, dpp_partner<0x141>(v));  // row_half_mirror
  if (lpr > 8) v = op(v, dpp_partner<0x140>(v));  // row_mirror
  if (lpr > 16) {
    float lower = v, upper = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
    v = op(lower, upper);
  }
  if (lpr > 32) {
    float lower = v, upper = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
    v = op(lower, upper);
  }
  return v;
}
__device__ inline float lanes_max(float v, int lpr) {
  return lanes_reduce(v, lpr, [](float a, float b) { return fmaxf(a, b); });
}
__device__ inline float lanes_sum(float v, int lpr) {
  return lanes_reduce(v, lpr, [](float a, float b) { return a + b; });
}

// float offset of unit u, relative to the first block of the row and to the lane's own offset (the same for every
// lane: the compiler keeps it in scalar registers)
__device__ inline int64_t unit_offset(int u, const RowGeom &g) {
  const int t = u >> g.nq_log2;
  const int q = u & ((1 << g.nq_log2) - 1);
  return ((int64_t)t << (2 * g.sbs_log2)) + q * 256;
}

// What this wave works on: `first` (float offset of the row's first block), `units` (float4 units per lane) and the
// task index are the same for all lanes and are computed from values the compiler knows to be wave-uniform, so
// the loops over units branch on scalar registers instead of masking lanes.
__device__ inline bool wave_task(const RowGeom &g, const int32_t *row_offsets, int64_t n_tasks, int64_t &first,
                                 int &units, int &lane_base) {
  // Workgroup b runs on XCD b % 8: each XCD takes a contiguous eighth of the tasks, so the waves that read
  // neighbouring KiB of the same blocks (the tasks of one block row) share one L2.
  const int64_t n_groups = (n_tasks + kWaves - 1) / kWaves, per_xcd = (n_groups + 7) >> 3;
  const int64_t group = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int64_t wave = group * kWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (group >= n_groups || wave >= n_tasks) return false;
  const int lane = threadIdx.x & 63;
  const int64_t r = wave >> g.groups_log2;
  const int grp = (int)(wave & ((1 << g.groups_log2) - 1));
  const int start = row_offsets[r];
  const int count = row_offsets[r + 1] - start;
  if (count <= 0) return false;
  first = (int64_t)start << (2 * g.sbs_log2);
  units = count << g.nq_log2;
  const int rows_per_wave = 64 / g.lpr;
  const int row_in_block = grp * rows_per_wave + lane / g.lpr;
  lane_base = (row_in_block << g.sbs_log2) + (lane % g.lpr) * 4;
  return true;
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// the result is written once and not read back by the kernel: the store bypasses the caches
__device__ inline void store_streaming(float *p, float4 o) {
  __builtin_nontemporal_store(f32x4_t{o.x, o.y, o.z, o.w}, reinterpret_cast<f32x4_t *>(p));
}

// e^(v - m) through the hardware's 2^x as 2^(v * log2(e) - m2) with m2 = m * log2(e): one fused multiply-add and
// one transcendental instruction per element.  The rounding of m2 is a factor common to every element of the
// row and cancels against the row sum; what is left is the rounding of the exponent's argument, a relative
// error of about |v - m| * 1e-7, far inside the 1e-5 the operation is held to.  (The library's expf costs ten
// times the instructions, which made the kernel compute-bound.)
constexpr float kLog2e = 1.44269504088896341f;
__device__ inline float exp_rel(float v, float m2) { return __builtin_amdgcn_exp2f(__builtin_fmaf(v, kLog2e, -m2)); }
__device__ inline float exp2_of(float d) { return __builtin_amdgcn_exp2f(d); }

// max(m, v.x, v.y, v.z, v.w) in two instructions.  fmaxf first quiets signalling NaNs (one more instruction per
// operand); here a NaN may come out either way: it reaches every output of the row through the exponentials.
__device__ inline float max_with(float m, float4 v) {
  float t;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(t) : "v"(v.x), "v"(v.y), "v"(v.z));
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(t) : "v"(t), "v"(v.w), "v"(m));
  return t;
}

// Loads units [0, units) of a row into v, four at a time: within a group of four the index is clamped to the last
// unit (a repeated load of a line just fetched) so that the group has no branch, and no load is followed by its
// use: all loads of the row are in flight together.  Entries at and beyond `units` hold copies of the last unit.
template <int N>
__device__ inline void load_row(float4 (&v)[N], const float *row, int units, const RowGeom &g) {
#pragma unroll
  for (int c = 0; c < N; c += 4) {
    if (c < units) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int u = c + j < units ? c + j : units - 1;
        v[c + j] = *reinterpret_cast<const float4 *>(row + unit_offset(u, g));
      }
    }
  }
}

// Units [u0, u0 + count) of a row, count <= N: the index is clamped to the last of them, so the loads have no
// branch between them; entries at and beyond `count` hold copies of the last unit.
constexpr int kChunk = 8;
template <int N>
__device__ inline void load_chunk(float4 (&v)[N], const float *row, int u0, int count, const RowGeom &g) {
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int u = u0 + (j < count ? j : count - 1);
    v[j] = *reinterpret_cast<const float4 *>(row + unit_offset(u, g));
  }
}

__global__ __launch_bounds__(64 * kWaves) void softmax_fwd_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                          const int32_t *__restrict__ row_offsets, int64_t n_tasks,
                                                          RowGeom g) {
  int64_t first;
  int units, lane_base;
  if (!wave_task(g, row_offsets, n_tasks, first, units, lane_base)) return;
  const float *xr = x + first + lane_base;
  float *orow = out + first + lane_base;

  if (units <= kMaxUnits) {
    float4 v[kMaxUnits];
    load_row(v, xr, units, g);
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < kMaxUnits; c += 4) {
      if (c < units) {  // the copies of the last unit change no maximum
#pragma unroll
        for (int j = 0; j < 4; ++j) m = max_with(m, v[c + j]);
      }
    }
    const float m2 = lanes_max(m, g.lpr) * kLog2e;
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < kMaxUnits; ++u) {
      if (u < units) {
        v[u].x = exp_rel(v[u].x, m2);
        v[u].y = exp_rel(v[u].y, m2);
        v[u].z = exp_rel(v[u].z, m2);
        v[u].w = exp_rel(v[u].w, m2);
        s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
      }
    }
    s = lanes_sum(s, g.lpr);
    const float inv = 1.f / s;  // one division per row, then products
#pragma unroll
    for (int u = 0; u < kMaxUnits; ++u) {
      if (u < units) {
        float4 o;
        o.x = v[u].x * inv;
        o.y = v[u].y * inv;
        o.z = v[u].z * inv;
        o.w = v[u].w * inv;
        store_streaming(orow + unit_offset(u, g), o);
      }
    }
    return;
  }

  // long rows: max pass and sum pass folded into one online pass, then the write pass; both in chunks of
  // kChunk units whose loads are all issued before the first one is used
  float m = -INFINITY, s = 0.f;
  for (int u0 = 0; u0 < units; u0 += kChunk) {
    const int count = units - u0 < kChunk ? units - u0 : kChunk;
    float4 v[kChunk];
    load_chunk(v, xr, u0, count, g);
    float mn = m;
#pragma unroll
    for (int j = 0; j < kChunk; ++j) mn = max_with(mn, v[j]);  // the copies of the last unit change no maximum
    if (mn != -INFINITY) {
      const float mn2 = mn * kLog2e;
      float add = 0.f;
#pragma unroll
      for (int j = 0; j < kChunk; ++j)
        if (j < count)
          add += (exp_rel(v[j].x, mn2) + exp_rel(v[j].y, mn2)) + (exp_rel(v[j].z, mn2) + exp_rel(v[j].w, mn2));
      s = s * exp2_of(m * kLog2e - mn2) + add;
    } else {
      bool any_nan = false;  // a maximum that dropped a NaN: keep it visible in the sum
#pragma unroll
      for (int j = 0; j < kChunk; ++j)
        any_nan |= v[j].x != v[j].x || v[j].y != v[j].y || v[j].z != v[j].z || v[j].w != v[j].w;
      if (any_nan) s = NAN;
    }
    m = mn;
  }
  const float mall = lanes_max(m, g.lpr);
  const float mall2 = mall * kLog2e;
  float part = (m == -INFINITY) ? ((s != s) ? s : 0.f) : s * exp2_of(m * kLog2e - mall2);
  const float sall = lanes_sum(part, g.lpr);
  const float inv_all = 1.f / sall;
  for (int u0 = 0; u0 < units; u0 += kChunk) {
    const int count = units - u0 < kChunk ? units - u0 : kChunk;
    float4 v[kChunk];
    load_chunk(v, xr, u0, count, g);
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      if (j < count) {
        float4 o;
        o.x = exp_rel(v[j].x, mall2) * inv_all;
        o.y = exp_rel(v[j].y, mall2) * inv_all;
        o.z = exp_rel(v[j].z, mall2) * inv_all;
        o.w = exp_rel(v[j].w, mall2) * inv_all;
        store_streaming(orow + unit_offset(u0 + j, g), o);
      }
    }
  }
}

__global__ __launch_bounds__(64 * kWaves) void softmax_bwd_kernel(const float *__restrict__ grad_out,
                                                          const float *__restrict__ y, float *__restrict__ grad_in,
                                                          const int32_t *__restrict__ row_offsets, int64_t n_tasks,
                                                          RowGeom g) {
  int64_t first;
  int units, lane_base;
  if (!wave_task(g, row_offsets, n_tasks, first, units, lane_base)) return;
  const float *gr = grad_out + first + lane_base;
  const float *yr = y + first + lane_base;
  float *dr = grad_in + first + lane_base;

  if (units <= kMaxUnits / 2) {
    constexpr int kU = kMaxUnits / 2;
    float4 yv[kU], gv[kU];
    load_row(yv, yr, units, g);
    load_row(gv, gr, units, g);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (u < units) s += (yv[u].x * gv[u].x + yv[u].y * gv[u].y) + (yv[u].z * gv[u].z + yv[u].w * gv[u].w);
    }
    s = lanes_sum(s, g.lpr);
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (u < units) {
        float4 o;
        o.x = yv[u].x * (gv[u].x - s);
        o.y = yv[u].y * (gv[u].y - s);
        o.z = yv[u].z * (gv[u].z - s);
        o.w = yv[u].w * (gv[u].w - s);
        store_streaming(dr + unit_offset(u, g), o);
      }
    }
    return;
  }

  if (units <= kMaxUnits) {
    // middle rows: y stays in registers, the gradient passes twice in chunks (once for the row's sum, once for the
    // result): 1.5 instead of 2 reads of the row's 2 x 16 bytes per element
    float4 yv[kMaxUnits];
    load_row(yv, yr, units, g);
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < kMaxUnits; c += kChunk) {
      if (c < units) {
        const int count = units - c < kChunk ? units - c : kChunk;
        float4 gv[kChunk];
        load_chunk(gv, gr, c, count, g);
#pragma unroll
        for (int j = 0; j < kChunk; ++j)
          if (j < count)
            s += (yv[c + j].x * gv[j].x + yv[c + j].y * gv[j].y) + (yv[c + j].z * gv[j].z + yv[c + j].w * gv[j].w);
      }
    }
    s = lanes_sum(s, g.lpr);
#pragma unroll
    for (int c = 0; c < kMaxUnits; c += kChunk) {
      if (c < units) {
        const int count = units - c < kChunk ? units - c : kChunk;
        float4 gv[kChunk];
        load_chunk(gv, gr, c, count, g);
#pragma unroll
        for (int j = 0; j < kChunk; ++j) {
          if (j < count) {
            float4 o;
            o.x = yv[c + j].x * (gv[j].x - s);
            o.y = yv[c + j].y * (gv[j].y - s);
            o.z = yv[c + j].z * (gv[j].z - s);
            o.w = yv[c + j].w * (gv[j].w - s);
            store_streaming(dr + unit_offset(c + j, g), o);
          }
        }
      }
    }
    return;
  }

  // long rows: two passes in chunks whose loads are all issued before the first one is used
  float s = 0.f;
  for (int u0 = 0; u0 < units; u0 += kChunk) {
    const int count = units - u0 < kChunk ? units - u0 : kChunk;
    float4 yv[kChunk], gv[kChunk];
    load_chunk(yv, yr, u0, count, g);
    load_chunk(gv, gr, u0, count, g);
#pragma unroll
    for (int j = 0; j < kChunk; ++j)
      if (j < count) s += (yv[j].x * gv[j].x + yv[j].y * gv[j].y) + (yv[j].z * gv[j].z + yv[j].w * gv[j].w);
  }
  s = lanes_sum(s, g.lpr);
  for (int u0 = 0; u0 < units; u0 += kChunk) {
    const int count = units - u0 < kChunk ? units - u0 : kChunk;
    float4 yv[kChunk], gv[kChunk];
    load_chunk(yv, yr, u0, count, g);
    load_chunk(gv, gr, u0, count, g);
#pragma unroll
    for (int j = 0; j < kChunk; ++j) {
      if (j < count) {
        float4 o;
        o.x = yv[j].x * (gv[j].x - s);
        o.y = yv[j].y * (gv[j].y - s);
        o.z = yv[j].z * (gv[j].z - s);
        o.w = yv[j].w * (gv[j].w - s);
        store_streaming(dr + unit_offset(u0 + j, g), o);
      }
    }
  }
}

int make_geom(const char *who, int sbs, RowGeom &g) {
  BSA_REQUIRE(sbs >= 16 && bsa::is_pow2(sbs), "%s: sbs must be a power of two >= 16 (got %d)", who, sbs);
  int l = 0;
  while ((1 << l) < sbs) ++l;
  g.sbs_log2 = l;
  g.lpr = sbs / 4 < 64 ? sbs / 4 : 64;
  int nq = sbs / 256 > 1 ? sbs / 256 : 1;
  g.nq_log2 = 0;
  while ((1 << g.nq_log2) < nq) ++g.nq_log2;
  g.groups_log2 = 0;
  while ((1 << g.groups_log2) < sbs * g.lpr / 64) ++g.groups_log2;
  return BSA_OK;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int bsa_softmax_fwd(const float *x, float *out, const int32_t *row_offsets, int64_t n_rows, int64_t nnz,
                               int sbs, bsa_stream_t stream) {
  RowGeom g;
  if (int rc = make_geom("bsa_softmax_fwd", sbs, g)) return rc;
  BSA_REQUIRE(n_rows >= 0 && nnz >= 0, "bsa_softmax_fwd: negative size");
  if (n_rows == 0 || nnz == 0) return BSA_OK;
  BSA_REQUIRE(x && out && row_offsets, "bsa_softmax_fwd: NULL pointer");
  BSA_REQUIRE(aligned16(x) && aligned16(out), "bsa_softmax_fwd: buffers must be 16-byte aligned");
  if (nnz > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_softmax_fwd: more than 2^31-1 blocks");
  const int64_t n_tasks = n_rows << g.groups_log2;
  const int64_t blocks = bsa::cdiv(bsa::cdiv(n_tasks, kWaves), 8) * 8;  // a whole number of workgroups per XCD
  if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_softmax_fwd: too many rows");
  softmax_fwd_kernel<<<(unsigned)blocks, 64 * kWaves, 0, bsa::as_stream(stream)>>>(x, out, row_offsets, n_tasks, g);
  return bsa::check_launch("softmax_fwd_kernel");
}

extern "C" int bsa_softmax_bwd(const float *grad_out, const float *y, float *grad_in, const int32_t *row_offsets,
                               int64_t n_rows, int64_t nnz, int sbs, bsa_stream_t stream) {
  RowGeom g;
  if (int rc = make_geom("bsa_softmax_bwd", sbs, g)) return rc;
  BSA_REQUIRE(n_rows >= 0 && nnz >= 0, "bsa_softmax_bwd: negative size");
  if (n_rows == 0 || nnz == 0) return BSA_OK;
  BSA_REQUIRE(grad_out && y && grad_in && row_offsets, "bsa_softmax_bwd: NULL pointer");
  BSA_REQUIRE(aligned16(grad_out) && aligned16(y) && aligned16(grad_in),
              "bsa_softmax_bwd: buffers must be 16-byte aligned");
  if (nnz > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_softmax_bwd: more than 2^31-1 blocks");
  const int64_t n_tasks = n_rows << g.groups_log2;
  const int64_t blocks = bsa::cdiv(bsa::cdiv(n_tasks, kWaves), 8) * 8;  // a whole number of workgroups per XCD
  if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_softmax_bwd: too many rows");
  softmax_bwd_kernel<<<(unsigned)blocks, 64 * kWaves, 0, bsa::as_stream(stream)>>>(grad_out, y, grad_in, row_offsets,
                                                                           n_tasks, g);
  return bsa::check_launch("softmax_bwd_kernel");
}
