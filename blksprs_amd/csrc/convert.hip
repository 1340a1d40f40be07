// Dense <-> compressed conversion: 16-byte vector copies, one thread per vector.
//
// A block row is sbs * elem_size bytes, a multiple of 16 for every supported
// (sbs >= 16, elem_size >= 1), so both directions move uint4 vectors and are
// independent of the element type.  Traffic: to_sparse reads and writes
// nnz*sbs*sbs*elem_size bytes; to_dense writes the whole dense array once and
// reads the active blocks once.
#include "common.h"

namespace {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// For a kernel that only reads: the load does not keep its lines in the caches (build_sparsity_layout gains
// 12 %).  The kernels that read and write lose 5 to 20 % with such loads and keep plain ones.
__device__ inline uint4 load_streaming(const uint4 *p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
  return uint4{v[0], v[1], v[2], v[3]};
}

// results that are written once and not read back by the kernel bypass the caches
__device__ inline void store_streaming(uint4 *p, uint4 v) {
  __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t *>(p));
}

// blocks[n][e][:] <- dense[b][r*sbs + e][c*sbs : (c+1)*sbs]
__global__ __launch_bounds__(256) void to_sparse_kernel(const uint4 *__restrict__ dense,
                                                        const int64_t *__restrict__ coords,
                                                        uint4 *__restrict__ blocks, int64_t n_vec,
                                                        int vec_per_row_log2, int sbs_log2, int64_t dense_row_vecs,
                                                        int64_t dense_batch_vecs) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int vec_per_block_log2 = vec_per_row_log2 + sbs_log2;
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_vec; g += stride) {
    const int64_t n = g >> vec_per_block_log2;
    const int64_t in_block = g & (((int64_t)1 << vec_per_block_log2) - 1);
    const int64_t e = in_block >> vec_per_row_log2;
    const int64_t q = in_block & (((int64_t)1 << vec_per_row_log2) - 1);
    const int64_t b = coords[n * 3 + 0];
    const int64_t r = coords[n * 3 + 1];
    const int64_t c = coords[n * 3 + 2];
    const int64_t src = b * dense_batch_vecs + ((r << sbs_log2) + e) * dense_row_vecs + (c << vec_per_row_log2) + q;
    store_streaming(blocks + g, dense[src]);
  }
}

// dense[b][row][:] <- blocks[packed[b, row/sbs, col/sbs]] or the fill pattern.  A thread owns one 16-byte
// column position in kDenseRows consecutive rows of the dense array (they lie in one block row, so one look-up
// serves them all); a wave writes 1 KiB of a row at a time.  The dense array is written once and not read
// back by this kernel: the stores bypass the caches.
constexpr int kDenseRows = 4;  // divides every sbs

__global__ __launch_bounds__(256) void to_dense_kernel(const u32x4_t *__restrict__ blocks,
                                                       const int64_t *__restrict__ packed,
                                                       u32x4_t *__restrict__ dense, int64_t nnz, int64_t C,
                                                       int64_t dense_row_vecs, int64_t row_groups,
                                                       int vec_per_row_log2, int sbs_log2, u32x4_t fill) {
  const int64_t col_vec = (int64_t)blockIdx.y * 256 + threadIdx.x;
  if (col_vec >= dense_row_vecs) return;
  const int64_t c = col_vec >> vec_per_row_log2;
  const int64_t q = col_vec & (((int64_t)1 << vec_per_row_log2) - 1);
  // a launch holds fewer than 2^32 threads: beyond 2^23 groups of rows a workgroup takes several
  for (int64_t group = blockIdx.x; group < row_groups; group += gridDim.x) {
    const int64_t row0 = group * kDenseRows;  // b * R * sbs + row
    const int64_t e0 = row0 & (((int64_t)1 << sbs_log2) - 1);
    const int64_t br = row0 >> sbs_log2;  // b * R + r
    const int64_t idx = packed[br * C + c];
    const bool active = idx >= 0 && idx < nnz;
    u32x4_t v[kDenseRows];
#pragma unroll
    for (int i = 0; i < kDenseRows; ++i) {
      v[i] = fill;
      if (active) v[i] = blocks[(((idx << sbs_log2) + e0 + i) << vec_per_row_log2) + q];
    }
#pragma unroll
    for (int i = 0; i < kDenseRows; ++i) __builtin_nontemporal_store(v[i], dense + (row0 + i) * dense_row_vecs + col_vec);
  }
}

// layout[b][r][c] = 1 if the sbs x sbs block (r, c) of dense[b] holds an element != 0.  One workgroup owns
// one block row (sbs dense rows) and a chunk of kLayoutVecs 16-byte vectors of every row: thread t owns the
// vectors t, t + 256, ... of the chunk in all sbs rows (every row read is one contiguous run), ORs the masked
// words of its column positions over the rows, and reports to the blocks its positions belong to.  `mask`
// clears the sign bits of floating-point elements: -0.0 equals 0, NaN does not.  Several threads (and, for
// very wide blocks, several workgroups) may report the same block: they all store the same 1.
constexpr int kLayoutPerThread = 4;
constexpr int kLayoutVecs = 256 * kLayoutPerThread;
constexpr int kLayoutRows = 16;  // element rows per workgroup

__global__ __launch_bounds__(256) void layout_from_dense_kernel(const uint4 *__restrict__ dense,
                                                                uint8_t *__restrict__ layout, int64_t row_vecs,
                                                                int sbs, int vec_per_row_log2, int64_t C, uint4 mask) {
  const int64_t block_row = blockIdx.x;  // b * R + r
  const int64_t chunk0 = (int64_t)blockIdx.y * kLayoutVecs;
  const uint4 *base = dense + block_row * sbs * row_vecs;
  uint32_t any[kLayoutPerThread] = {0u, 0u, 0u, 0u};
  // blockIdx.z takes kLayoutRows of the block row's element rows (a workgroup that walked all of them would be
  // one long chain of load rounds; the workgroups of one block row all store the same 1).  sbs is a multiple
  // of 4: four rows (16 loads) are in flight at a time
  const int e_begin = blockIdx.z * kLayoutRows, e_end = e_begin + kLayoutRows < sbs ? e_begin + kLayoutRows : sbs;
  for (int e0 = e_begin; e0 < e_end; e0 += 4) {
    uint4 w[4][kLayoutPerThread];
#pragma unroll
    for (int de = 0; de < 4; ++de) {
      const uint4 *row = base + (int64_t)(e0 + de) * row_vecs;
#pragma unroll
      for (int i = 0; i < kLayoutPerThread; ++i) {
        const int64_t v = chunk0 + threadIdx.x + 256 * i;
        w[de][i] = uint4{0u, 0u, 0u, 0u};
        if (v < row_vecs) w[de][i] = load_streaming(row + v);
      }
    }
#pragma unroll
    for (int de = 0; de < 4; ++de)
#pragma unroll
      for (int i = 0; i < kLayoutPerThread; ++i)
        any[i] |= (w[de][i].x & mask.x) | (w[de][i].y & mask.y) | (w[de][i].z & mask.z) | (w[de][i].w & mask.w);
  }
#pragma unroll
  for (int i = 0; i < kLayoutPerThread; ++i) {
    const int64_t v = chunk0 + threadIdx.x + 256 * i;
    if (v < row_vecs && any[i]) layout[block_row * C + (v >> vec_per_row_log2)] = 1;
  }
}

// out[o] = transpose of blocks[packed[flat index of coords[o] in the (B, R, C) output layout]] (zeros where that
// entry is negative or out of range): the gather of flow_pull fused with the element transposition.  One
// workgroup moves one 64 x 64 (or sbs x sbs for smaller blocks) tile of elements through LDS: rows in, columns
// out, both sides touching consecutive elements of a row.
template <typename E>
__global__ __launch_bounds__(256) void transpose_blocks_kernel(const E *__restrict__ blocks,
                                                               const int64_t *__restrict__ coords,
                                                               const int64_t *__restrict__ packed,
                                                               E *__restrict__ out, int64_t n_src, int64_t R,
                                                               int64_t C, int sbs, int tiles_per_side) {
  __shared__ E tile[64][65];
  const int T = sbs < 64 ? sbs : 64;
  const int64_t o = blockIdx.x / (tiles_per_side * tiles_per_side);
  const int t_id = blockIdx.x % (tiles_per_side * tiles_per_side);
  const int tr = t_id / tiles_per_side, tc = t_id % tiles_per_side;  // tile of the OUTPUT block
  const int64_t b = coords[o * 3 + 0], r = coords[o * 3 + 1], c = coords[o * 3 + 2];
  const int64_t flat = (b * R + r) * C + c;
  int64_t src = -1;
  if (r >= 0 && r < R && c >= 0 && c < C && b >= 0) src = packed[flat];
  const bool valid = src >= 0 && src < n_src;
  const int col = threadIdx.x % T, row0 = threadIdx.x / T, rows_per_pass = 256 / T;
  if (valid) {
    // input tile (tc, tr) of the source block: rows 64 tc .., columns 64 tr ..
    const E *in = blocks + src * sbs * sbs + ((int64_t)tc * T) * sbs + (int64_t)tr * T;
    for (int row = row0; row < T; row += rows_per_pass) tile[row][col] = in[(int64_t)row * sbs + col];
  }
  __syncthreads();
  E *dst = out + o * sbs * sbs + ((int64_t)tr * T) * sbs + (int64_t)tc * T;
  for (int row = row0; row < T; row += rows_per_pass) dst[(int64_t)row * sbs + col] = valid ? tile[col][row] : E(0);
}

// The same operation for 2-byte elements and sbs >= 64, moving 16-byte vectors on both sides.  A workgroup of
// four waves stages one 64 x 64 tile of the source block (8 KiB) in LDS, turns it with the transposing LDS read
// (sixteen lanes that point at a 4 x 16 patch of elements each get one column of it), parks the turned vectors
// in a second tile and stores that row by row, so every global access is a full 128-byte row.
using i16x4_t = short __attribute__((ext_vector_type(4)));
using u32x2_t = uint32_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x2_t read_turned(const char *p) {
  const i16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t *)p);
  return __builtin_bit_cast(u32x2_t, v);
}

// XOR on the 16-byte chunk index of row r of the staged tile: a transposing read serves 32 lanes at a time, rows
// r .. r + 3 (r a multiple of 4) with 64 consecutive bytes of each, and two 128-byte rows span the 64 banks
// once, so rows r and r + 2 keep their 64 bytes in different halves of the row.
__device__ __forceinline__ int turn_swizzle(int r) { return ((r >> 1) & 1) << 2; }

__global__ __launch_bounds__(256) void transpose_blocks16_kernel(const uint16_t *__restrict__ blocks,
                                                                 const int64_t *__restrict__ coords,
                                                                 const int64_t *__restrict__ packed,
                                                                 uint16_t *__restrict__ out, int64_t n_src,
                                                                 int64_t R, int64_t C, int sbs, int tiles_per_side) {
  __shared__ __attribute__((aligned(16))) char in_tile[64 * 128];
  __shared__ __attribute__((aligned(16))) char out_tile[64 * 128];
  const int64_t o = blockIdx.x / (tiles_per_side * tiles_per_side);
  const int t_id = blockIdx.x % (tiles_per_side * tiles_per_side);
  const int tr = t_id / tiles_per_side, tc = t_id % tiles_per_side;  // tile of the OUTPUT block
  const int64_t b = coords[o * 3 + 0], r = coords[o * 3 + 1], c = coords[o * 3 + 2];
  int64_t src = -1;
  if (r >= 0 && r < R && c >= 0 && c < C && b >= 0) src = packed[(b * R + r) * C + c];
  const bool valid = src >= 0 && src < n_src;  // uniform over the workgroup
  const int t = threadIdx.x;
  const int64_t row_bytes = (int64_t)sbs * 2;
  char *dst = reinterpret_cast<char *>(out) + o * sbs * row_bytes + ((int64_t)tr * 64) * row_bytes + tc * 128;
  if (!valid) {
    for (int v = t; v < 512; v += 256) *reinterpret_cast<uint4 *>(dst + (v >> 3) * row_bytes + (v & 7) * 16) = uint4{0, 0, 0, 0};
    return;
  }
  // source tile (tc, tr): rows 64 tc .., columns 64 tr ..
  const char *in = reinterpret_cast<const char *>(blocks) + src * sbs * row_bytes + ((int64_t)tc * 64) * row_bytes + tr * 128;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int v = t + 256 * i, row = v >> 3, chunk = v & 7;
    const uint4 w = *reinterpret_cast<const uint4 *>(in + row * row_bytes + chunk * 16);
    *reinterpret_cast<uint4 *>(in_tile + row * 128 + ((chunk ^ turn_swizzle(row)) << 4)) = w;
  }
  __syncthreads();
  // wave w turns source rows 16 w .. 16 w + 15; lane group g: rows + 8 (g / 2), columns + 16 (g % 2)
  const int wave = t >> 6, lane = t & 63, g = lane >> 4, ls = lane & 15;
#pragma unroll
  for (int cb = 0; cb < 2; ++cb) {
    const int r0 = 16 * wave + 8 * (g >> 1);
    const int col0 = 32 * cb + 16 * (g & 1);
    u32x2_t half[2];
#pragma unroll
    for (int rd = 0; rd < 2; ++rd) {
      const int rs = r0 + 4 * rd + (ls >> 2);
      const int col = col0 + 4 * (ls & 3);
      half[rd] = read_turned(in_tile + rs * 128 + (((col >> 3) ^ turn_swizzle(rs)) << 4) + ((col & 4) << 1));
    }
    // this lane now holds source[r0 .. r0 + 7][col0 + ls] = output row col0 + ls, columns r0 .. r0 + 7
    *reinterpret_cast<uint4 *>(out_tile + (col0 + ls) * 128 + (r0 >> 3) * 16) =
        uint4{half[0][0], half[0][1], half[1][0], half[1][1]};
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int v = t + 256 * i, row = v >> 3, chunk = v & 7;
    store_streaming(reinterpret_cast<uint4 *>(dst + row * row_bytes + chunk * 16),
                    *reinterpret_cast<const uint4 *>(out_tile + row * 128 + chunk * 16));
  }
}

int ilog2(int64_t v) {
  int l = 0;
  while (((int64_t)1 << l) < v) ++l;
  return l;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_block_shape(const char *who, int sbs, int elem_size) {
  BSA_REQUIRE(sbs >= 16 && bsa::is_pow2(sbs), "%s: sbs must be a power of two >= 16 (got %d)", who, sbs);
  BSA_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8,
              "%s: element size %d not in {1,2,4,8}", who, elem_size);
  return BSA_OK;
}

unsigned copy_grid(int64_t n_vec) {
  // enough resident threads to cover the memory latency of 256 CUs; the grid-stride loop takes the rest
  int64_t blocks = bsa::cdiv(n_vec, 256);
  const int64_t cap = 256 * 32;
  return (unsigned)(blocks < cap ? blocks : cap);
}

}  // namespace

extern "C" int bsa_to_sparse(const void *dense, const int64_t *coords, void *blocks, int64_t nnz, int64_t rows,
                             int64_t cols, int sbs, int elem_size, bsa_stream_t stream) {
  if (int rc = check_block_shape("bsa_to_sparse", sbs, elem_size)) return rc;
  BSA_REQUIRE(nnz >= 0 && rows >= 0 && cols >= 0, "bsa_to_sparse: negative size");
  BSA_REQUIRE(rows % sbs == 0 && cols % sbs == 0, "bsa_to_sparse: dense sizes not divisible by sbs");
  if (nnz == 0) return BSA_OK;
  BSA_REQUIRE(dense && coords && blocks, "bsa_to_sparse: NULL pointer");
  BSA_REQUIRE(aligned16(dense) && aligned16(blocks), "bsa_to_sparse: buffers must be 16-byte aligned");
  const int vec_per_row = sbs * elem_size / 16;
  const int64_t n_vec = nnz * sbs * vec_per_row;
  const int64_t dense_row_vecs = cols * elem_size / 16;
  to_sparse_kernel<<<copy_grid(n_vec), 256, 0, bsa::as_stream(stream)>>>(
      static_cast<const uint4 *>(dense), coords, static_cast<uint4 *>(blocks), n_vec, ilog2(vec_per_row),
      ilog2(sbs), dense_row_vecs, rows * dense_row_vecs);
  return bsa::check_launch("to_sparse_kernel");
}

extern "C" int bsa_to_dense(const void *blocks, const int64_t *packed, void *dense, int64_t B, int64_t R, int64_t C,
                            int64_t nnz, int sbs, int elem_size, uint64_t fill_bits, bsa_stream_t stream) {
  if (int rc = check_block_shape("bsa_to_dense", sbs, elem_size)) return rc;
  BSA_REQUIRE(B >= 0 && R >= 0 && C >= 0 && nnz >= 0, "bsa_to_dense: negative size");
  const int vec_per_row = sbs * elem_size / 16;
  const int64_t n_vec = B * R * sbs * C * vec_per_row;
  if (n_vec == 0) return BSA_OK;
  BSA_REQUIRE(packed && dense && (nnz == 0 || blocks), "bsa_to_dense: NULL pointer");
  BSA_REQUIRE(aligned16(dense) && aligned16(blocks), "bsa_to_dense: buffers must be 16-byte aligned");
  // replicate the element pattern across 16 bytes
  uint64_t pat = fill_bits;
  if (elem_size < 8) pat &= ((uint64_t)1 << (8 * elem_size)) - 1;
  for (int w = elem_size; w < 8; w *= 2) pat |= pat << (8 * w);
  const u32x4_t fill{(uint32_t)(pat & 0xffffffffu), (uint32_t)(pat >> 32), (uint32_t)(pat & 0xffffffffu),
                     (uint32_t)(pat >> 32)};
  const int64_t dense_row_vecs = C * vec_per_row;
  const int64_t row_groups = B * R * sbs / kDenseRows;
  const int64_t col_groups = bsa::cdiv(dense_row_vecs, 256);
  BSA_REQUIRE(col_groups <= 65535, "bsa_to_dense: dense rows too long for one launch");
  // fewer than 2^32 threads per launch (HIP refuses more): the workgroups of a column stride over the rows
  int64_t grid_rows = ((int64_t)1 << 23) / col_groups;
  if (grid_rows < 1) grid_rows = 1;
  if (grid_rows > row_groups) grid_rows = row_groups;
  to_dense_kernel<<<dim3((unsigned)grid_rows, (unsigned)col_groups), 256, 0, bsa::as_stream(stream)>>>(
      static_cast<const u32x4_t *>(blocks), packed, static_cast<u32x4_t *>(dense), nnz, C, dense_row_vecs, row_groups,
      ilog2(vec_per_row), ilog2(sbs), fill);
  return bsa::check_launch("to_dense_kernel");
}

extern "C" int bsa_layout_from_dense(const void *dense, uint8_t *layout, int64_t B, int64_t R, int64_t C, int sbs,
                                     int elem_size, int is_float, bsa_stream_t stream) {
  if (int rc = check_block_shape("bsa_layout_from_dense", sbs, elem_size)) return rc;
  BSA_REQUIRE(B >= 0 && R >= 0 && C >= 0, "bsa_layout_from_dense: negative size");
  BSA_REQUIRE(!is_float || elem_size >= 2, "bsa_layout_from_dense: no floating-point type of 1 byte");
  if (B * R * C == 0) return BSA_OK;
  BSA_REQUIRE(dense && layout, "bsa_layout_from_dense: NULL pointer");
  BSA_REQUIRE(aligned16(dense), "bsa_layout_from_dense: buffer must be 16-byte aligned");
  BSA_REQUIRE(B * R < 0x7fffffffLL, "bsa_layout_from_dense: too many block rows");
  const int vec_per_row = sbs * elem_size / 16;
  const int64_t row_vecs = C * vec_per_row;
  const int64_t chunks = bsa::cdiv(row_vecs, kLayoutVecs);
  BSA_REQUIRE(chunks <= 65535, "bsa_layout_from_dense: rows too long");
  uint4 mask{0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  if (is_float) {
    const uint32_t m = elem_size == 2 ? 0x7fff7fffu : 0x7fffffffu;
    mask = uint4{m, m, m, m};
    if (elem_size == 8) mask = uint4{0xffffffffu, 0x7fffffffu, 0xffffffffu, 0x7fffffffu};  // sign in the high word
  }
  layout_from_dense_kernel<<<dim3((unsigned)(B * R), (unsigned)chunks, (unsigned)((sbs + kLayoutRows - 1) / kLayoutRows)),
                             256, 0, bsa::as_stream(stream)>>>(
      static_cast<const uint4 *>(dense), layout, row_vecs, sbs, ilog2(vec_per_row), C, mask);
  return bsa::check_launch("layout_from_dense_kernel");
}

extern "C" int bsa_transpose_blocks(const void *blocks, const int64_t *coords, const int64_t *packed, void *out,
                                    int64_t nnz_out, int64_t nnz_in, int64_t B, int64_t R, int64_t C, int sbs,
                                    int elem_size, bsa_stream_t stream) {
  if (int rc = check_block_shape("bsa_transpose_blocks", sbs, elem_size)) return rc;
  BSA_REQUIRE(nnz_out >= 0 && nnz_in >= 0 && B >= 0 && R >= 0 && C >= 0, "bsa_transpose_blocks: negative size");
  if (nnz_out == 0) return BSA_OK;
  BSA_REQUIRE(coords && packed && out && (nnz_in == 0 || blocks), "bsa_transpose_blocks: NULL pointer");
  const int tiles = sbs <= 64 ? 1 : sbs / 64;
  const int64_t grid = nnz_out * tiles * tiles;
  BSA_REQUIRE(grid < ((int64_t)1 << 24), "bsa_transpose_blocks: too many tiles for one launch (2^24 at most)");
  hipStream_t s = bsa::as_stream(stream);
  if (elem_size == 2 && sbs >= 64 && aligned16(blocks) && aligned16(out)) {
    transpose_blocks16_kernel<<<(unsigned)grid, 256, 0, s>>>(static_cast<const uint16_t *>(blocks), coords, packed,
                                                             static_cast<uint16_t *>(out), nnz_in, R, C, sbs, tiles);
    return bsa::check_launch("transpose_blocks16_kernel");
  }
#define BSA_TR_LAUNCH(E)                                                                                          \
  transpose_blocks_kernel<E><<<(unsigned)grid, 256, 0, s>>>(static_cast<const E *>(blocks), coords, packed,       \
                                                            static_cast<E *>(out), nnz_in, R, C, sbs, tiles)
  switch (elem_size) {
    case 1: BSA_TR_LAUNCH(uint8_t); break;
    case 2: BSA_TR_LAUNCH(uint16_t); break;
    case 4: BSA_TR_LAUNCH(uint32_t); break;
    default: BSA_TR_LAUNCH(uint64_t); break;
  }
#undef BSA_TR_LAUNCH
  return bsa::check_launch("transpose_blocks_kernel");
}
