// Row-wise reductions (sum, max) over the active blocks of a block row, and the row-wise add that
// broadcasts one value per element row back over those blocks.  fp32, fp16 and bf16.
//
// The blocks of one block row are consecutive in the compressed tensor (row-major block order), so a
// row is `count` whole blocks starting at row_offsets[r].  One wavefront owns a group of element rows of
// one block row and reads them with one 16-byte vector per lane: the 64 lanes cover 1 KiB of consecutive
// elements of a block (1024 / (sbs * elem) element rows), so every wave load is one contiguous KiB.
// The reduction runs in fp32, first down the blocks inside a lane, then across the lanes of an element
// row (xor shuffles): no atomics, the result does not depend on the launch order, and it is rounded to
// the element type once.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

struct RowGeom {
  int sbs_log2;
  int vec_log2;   // elements per 16-byte vector, as log2
  int lpr;        // lanes per element row = min(64, vectors per row)
  int nq_log2;    // vectors per lane per block row pass = max(1, vectors per row / 64), as log2
  int groups;     // wave tasks per block row = max(1, sbs * lpr / 64)
};

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int kPerVec = 4;
  __device__ static float load(const uint4 &v, int i) { return __uint_as_float((&v.x)[i]); }
  __device__ static void store(uint4 &v, int i, float f) { (&v.x)[i] = __float_as_uint(f); }
};
template <> struct Elem<__half> {
  static constexpr int kPerVec = 8;
  __device__ static float load(const uint4 &v, int i) {
    const uint32_t w = (&v.x)[i >> 1];
    return __half2float(__ushort_as_half((unsigned short)((i & 1) ? (w >> 16) : (w & 0xffffu))));
  }
  __device__ static void store(uint4 &v, int i, float f) {
    const uint32_t h = __half_as_ushort(__float2half_rn(f));
    uint32_t &w = (&v.x)[i >> 1];
    w = (i & 1) ? ((w & 0x0000ffffu) | (h << 16)) : ((w & 0xffff0000u) | h);
  }
};
template <> struct Elem<__hip_bfloat16> {
  static constexpr int kPerVec = 8;
  __device__ static float load(const uint4 &v, int i) {
    const uint32_t w = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  __device__ static uint32_t round(float f) {  // round to nearest even; NaN stays NaN
    const uint32_t u = __float_as_uint(f);
    if (f != f) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  }
  __device__ static void store(uint4 &v, int i, float f) {
    const uint32_t h = round(f);
    uint32_t &w = (&v.x)[i >> 1];
    w = (i & 1) ? ((w & 0x0000ffffu) | (h << 16)) : ((w & 0xffff0000u) | h);
  }
};

constexpr int kOpSum = 0, kOpMax = 1;

// out[packed_out[r]][e][0] = reduction of element row e over the blocks of block row r; the other columns of a
// square output block hold the neutral element (0 for the sum, -inf for the maximum).  A maximum over a row that
// holds a NaN is NaN.
template <typename T, int OP>
__global__ __launch_bounds__(256) void row_reduce_kernel(const uint4 *__restrict__ x, T *__restrict__ out,
                                                         const int32_t *__restrict__ row_offsets,
                                                         const int64_t *__restrict__ packed_out, int64_t n_tasks,
                                                         int64_t n_out, int slice_only, RowGeom g) {
  using E = Elem<T>;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wave >= n_tasks) return;
  const int lane = threadIdx.x & 63;
  const int64_t r = wave / g.groups;
  const int grp = (int)(wave % g.groups);
  const int start = row_offsets[r];
  const int count = row_offsets[r + 1] - start;
  if (count <= 0) return;
  const int64_t k = packed_out[r];
  if (k < 0 || k >= n_out) return;
  const int rows_per_wave = 64 / g.lpr;
  const int row_in_block = grp * rows_per_wave + lane / g.lpr;
  if (row_in_block >= (1 << g.sbs_log2)) return;  // a block smaller than 1 KiB leaves whole rows of lanes idle
  const int vecs_per_row_log2 = g.sbs_log2 - g.vec_log2;
  const int64_t block_vecs = (int64_t)1 << (g.sbs_log2 + vecs_per_row_log2);
  const uint4 *src = x + (int64_t)start * block_vecs + ((int64_t)row_in_block << vecs_per_row_log2) + lane % g.lpr;
  const int nq = 1 << g.nq_log2;

  float acc[4];
  bool has_nan = false;
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = OP == kOpSum ? 0.f : -INFINITY;
  auto fold = [&](const uint4 &v, float &a) {
#pragma unroll
    for (int i = 0; i < E::kPerVec; ++i) {
      const float f = E::load(v, i);
      if (OP == kOpSum) {
        a += f;
      } else {
        a = fmaxf(a, f);
        has_nan |= f != f;
      }
    }
  };
  const int units = count << g.nq_log2;  // vectors of this lane in the whole block row
  auto unit_ptr = [&](int u) { return src + (int64_t)(u >> g.nq_log2) * block_vecs + (u & (nq - 1)) * 64; };
  int u = 0;
  for (; u + 4 <= units; u += 4) {
    uint4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = *unit_ptr(u + i);
#pragma unroll
    for (int i = 0; i < 4; ++i) fold(v[i], acc[i]);
  }
  for (; u < units; ++u) {
    const uint4 v = *unit_ptr(u);
    fold(v, acc[0]);
  }
  float a = OP == kOpSum ? (acc[0] + acc[1]) + (acc[2] + acc[3]) : fmaxf(fmaxf(acc[0], acc[1]), fmaxf(acc[2], acc[3]));
  for (int d = 1; d < g.lpr; d <<= 1) {
    const float other = __shfl_xor(a, d);
    a = OP == kOpSum ? a + other : fmaxf(a, other);
  }
  if (OP == kOpMax) {
    // a row's lanes agree on whether any of them saw a NaN
    const unsigned long long votes = __ballot(has_nan);
    const int first_lane = lane - lane % g.lpr;
    const unsigned long long row_mask = (g.lpr == 64 ? ~0ull : ((1ull << g.lpr) - 1)) << first_lane;
    if (votes & row_mask) a = NAN;
  }

  if (slice_only) {
    if (lane % g.lpr == 0) {
      uint4 one{0, 0, 0, 0};
      E::store(one, 0, a);
      T *dst = out + (k << g.sbs_log2) + row_in_block;
      if (sizeof(T) == 4) *reinterpret_cast<uint32_t *>(dst) = one.x;
      else *reinterpret_cast<uint16_t *>(dst) = (uint16_t)(one.x & 0xffffu);
    }
    return;
  }
  uint4 fill{0, 0, 0, 0};
  if (OP == kOpMax) {
#pragma unroll
    for (int i = 0; i < E::kPerVec; ++i) E::store(fill, i, -INFINITY);
  }
  uint4 *dst = reinterpret_cast<uint4 *>(out) + k * block_vecs + ((int64_t)row_in_block << vecs_per_row_log2) +
               lane % g.lpr;
  for (int q = 0; q < nq; ++q) {
    uint4 v = fill;
    if (q == 0 && lane % g.lpr == 0) E::store(v, 0, a);
    dst[q * 64] = v;
  }
}

// out[n][e][:] = x[n][e][:] + y[packed_rows[b * R + r]][e][0] for block n = (b, r, c); blocks whose row has no
// entry in y are left zero.  Grid-stride loop over the 16-byte vectors of x.
template <typename T>
__global__ __launch_bounds__(256) void row_add_kernel(const uint4 *__restrict__ x, const int64_t *__restrict__ coords,
                                                      const int64_t *__restrict__ packed_rows,
                                                      const T *__restrict__ y, uint4 *__restrict__ out, int64_t n_vec,
                                                      int64_t n_y, int64_t B, int64_t R, int y_cols, int sbs_log2,
                                                      int vecs_per_row_log2) {
  using E = Elem<T>;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int block_vecs_log2 = sbs_log2 + vecs_per_row_log2;
  for (int64_t gi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; gi < n_vec; gi += stride) {
    const int64_t n = gi >> block_vecs_log2;
    const int64_t e = (gi & (((int64_t)1 << block_vecs_log2) - 1)) >> vecs_per_row_log2;
    const int64_t b = coords[n * 3 + 0], r = coords[n * 3 + 1];
    int64_t k = -1;
    if (b >= 0 && b < B && r >= 0 && r < R) k = packed_rows[b * R + r];
    uint4 v{0, 0, 0, 0};
    if (k >= 0 && k < n_y) {
      uint4 yv{0, 0, 0, 0};
      const T *yp = y + ((k << sbs_log2) + e) * y_cols;
      if (sizeof(T) == 4) yv.x = *reinterpret_cast<const uint32_t *>(yp);
      else yv.x = *reinterpret_cast<const uint16_t *>(yp);
      const float add = E::load(yv, 0);
      const uint4 xv = x[gi];
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i) E::store(v, i, E::load(xv, i) + add);
    }
    // written once, not read back here: bypass the caches
    __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t *>(out + gi));
  }
}

int ilog2(int64_t v) {
  int l = 0;
  while (((int64_t)1 << l) < v) ++l;
  return l;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int make_geom(const char *who, int sbs, int dtype, RowGeom &g) {
  BSA_REQUIRE(sbs >= 16 && bsa::is_pow2(sbs), "%s: sbs must be a power of two >= 16 (got %d)", who, sbs);
  BSA_REQUIRE(dtype == BSA_F32 || dtype == BSA_F16 || dtype == BSA_BF16, "%s: unknown dtype %d", who, dtype);
  const int per_vec = dtype == BSA_F32 ? 4 : 8;
  const int vecs_per_row = sbs / per_vec;
  g.sbs_log2 = ilog2(sbs);
  g.vec_log2 = ilog2(per_vec);
  g.lpr = vecs_per_row < 64 ? vecs_per_row : 64;
  g.nq_log2 = ilog2(vecs_per_row <= 64 ? 1 : vecs_per_row / 64);
  g.groups = sbs * g.lpr >= 64 ? sbs * g.lpr / 64 : 1;
  return BSA_OK;
}

template <typename T>
void launch_reduce(int op, unsigned blocks, hipStream_t s, const void *x, void *out, const int32_t *row_offsets,
                   const int64_t *packed_out, int64_t n_tasks, int64_t n_out, int slice_only, const RowGeom &g) {
  if (op == kOpSum)
    row_reduce_kernel<T, kOpSum><<<blocks, 256, 0, s>>>(static_cast<const uint4 *>(x), static_cast<T *>(out),
                                                        row_offsets, packed_out, n_tasks, n_out, slice_only, g);
  else
    row_reduce_kernel<T, kOpMax><<<blocks, 256, 0, s>>>(static_cast<const uint4 *>(x), static_cast<T *>(out),
                                                        row_offsets, packed_out, n_tasks, n_out, slice_only, g);
}

}  // namespace

extern "C" int bsa_row_reduce(const void *x, const int32_t *row_offsets, const int64_t *packed_out, void *out,
                              int64_t n_rows, int64_t n_out, int64_t nnz, int sbs, int dtype, int op, int slice_only,
                              bsa_stream_t stream) {
  RowGeom g;
  if (int rc = make_geom("bsa_row_reduce", sbs, dtype, g)) return rc;
  BSA_REQUIRE(op == kOpSum || op == kOpMax, "bsa_row_reduce: op must be 0 (sum) or 1 (max), got %d", op);
  BSA_REQUIRE(n_rows >= 0 && n_out >= 0 && nnz >= 0, "bsa_row_reduce: negative size");
  if (n_rows == 0 || n_out == 0 || nnz == 0) return BSA_OK;
  BSA_REQUIRE(x && row_offsets && packed_out && out, "bsa_row_reduce: NULL pointer");
  BSA_REQUIRE(aligned16(x) && (slice_only || aligned16(out)), "bsa_row_reduce: buffers must be 16-byte aligned");
  if (nnz > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_row_reduce: more than 2^31-1 blocks");
  const int64_t n_tasks = n_rows * g.groups;
  const int64_t blocks = bsa::cdiv(n_tasks, 4);
  if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_row_reduce: too many rows");
  hipStream_t s = bsa::as_stream(stream);
  switch (dtype) {
    case BSA_F32: launch_reduce<float>(op, (unsigned)blocks, s, x, out, row_offsets, packed_out, n_tasks, n_out, slice_only, g); break;
    case BSA_F16: launch_reduce<__half>(op, (unsigned)blocks, s, x, out, row_offsets, packed_out, n_tasks, n_out, slice_only, g); break;
    default: launch_reduce<__hip_bfloat16>(op, (unsigned)blocks, s, x, out, row_offsets, packed_out, n_tasks, n_out, slice_only, g); break;
  }
  return bsa::check_launch("row_reduce_kernel");
}

extern "C" int bsa_row_add(const void *x, const int64_t *coords, const int64_t *packed_rows, const void *y, void *out,
                           int64_t nnz, int64_t n_y, int64_t B, int64_t R, int y_cols, int sbs, int dtype,
                           bsa_stream_t stream) {
  RowGeom g;
  if (int rc = make_geom("bsa_row_add", sbs, dtype, g)) return rc;
  BSA_REQUIRE(nnz >= 0 && n_y >= 0 && B >= 0 && R >= 0, "bsa_row_add: negative size");
  BSA_REQUIRE(y_cols == 1 || y_cols == sbs, "bsa_row_add: y must have 1 or sbs columns (got %d)", y_cols);
  if (nnz == 0) return BSA_OK;
  BSA_REQUIRE(x && coords && packed_rows && out && (n_y == 0 || y), "bsa_row_add: NULL pointer");
  BSA_REQUIRE(aligned16(x) && aligned16(out), "bsa_row_add: buffers must be 16-byte aligned");
  const int vecs_per_row_log2 = g.sbs_log2 - g.vec_log2;
  const int64_t n_vec = nnz << (g.sbs_log2 + vecs_per_row_log2);
  int64_t blocks = bsa::cdiv(n_vec, 256);
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipStream_t s = bsa::as_stream(stream);
#define BSA_ROW_ADD(T)                                                                                            \
  row_add_kernel<T><<<(unsigned)blocks, 256, 0, s>>>(static_cast<const uint4 *>(x), coords, packed_rows,          \
                                                     static_cast<const T *>(y), static_cast<uint4 *>(out), n_vec, \
                                                     n_y, B, R, y_cols, g.sbs_log2, vecs_per_row_log2)
  switch (dtype) {
    case BSA_F32: BSA_ROW_ADD(float); break;
    case BSA_F16: BSA_ROW_ADD(__half); break;
    default: BSA_ROW_ADD(__hip_bfloat16); break;
  }
#undef BSA_ROW_ADD
  return bsa::check_launch("row_add_kernel");
}
