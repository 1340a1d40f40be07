// Work orders of the matmul kernels, built on the device (integer only): the order in which the tile kernel takes
// the output blocks, and the table by which the row kernel hands parts of block rows to workgroups.  Both are a
// stable sort of small integers by a 64-bit key that a kernel computes from tables already on the device, so no
// count is read back and the host never waits.  The sort is rocPRIM's radix sort (through hipCUB); its scratch
// comes from the caller like every other scratch of this library.  Neither order has a counterpart in the
// reference, whose kernels take output blocks in launch order (blksprs/ops/matmul.py:88-128); they only change
// which blocks are in flight together, never a result.
#include "common.h"

#include <hipcub/device/device_radix_sort.hpp>

namespace {

constexpr int kThreads = 256;
constexpr int kXcds = 8;

// scratch layout for n items: keys in, keys out (uint64 each), values in, values out (int32 each), then the sort's own
struct SortScratch {
  uint64_t *keys_in, *keys_out;
  int32_t *vals_in, *vals_out;
  void *temp;
  size_t temp_bytes;
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

size_t sort_temp_bytes(int64_t n) {
  size_t bytes = 0;
  // a size query: nothing is launched
  (void)hipcub::DeviceRadixSort::SortPairs(nullptr, bytes, static_cast<const uint64_t *>(nullptr),
                                           static_cast<uint64_t *>(nullptr), static_cast<const int32_t *>(nullptr),
                                           static_cast<int32_t *>(nullptr), (int)n, 0, 64, nullptr);
  return bytes;
}

size_t scratch_bytes(int64_t n) {
  const int64_t m = n > 0 ? n : 1;
  return 2 * align256(m * sizeof(uint64_t)) + 2 * align256(m * sizeof(int32_t)) + align256(sort_temp_bytes(m));
}

SortScratch carve(void *workspace, int64_t n) {
  const int64_t m = n > 0 ? n : 1;
  char *p = static_cast<char *>(workspace);
  SortScratch s;
  s.keys_in = reinterpret_cast<uint64_t *>(p);
  p += align256(m * sizeof(uint64_t));
  s.keys_out = reinterpret_cast<uint64_t *>(p);
  p += align256(m * sizeof(uint64_t));
  s.vals_in = reinterpret_cast<int32_t *>(p);
  p += align256(m * sizeof(int32_t));
  s.vals_out = reinterpret_cast<int32_t *>(p);
  p += align256(m * sizeof(int32_t));
  s.temp = p;
  s.temp_bytes = sort_temp_bytes(m);
  return s;
}

int sort_pairs(const SortScratch &s, int64_t n, hipStream_t stream) {
  size_t bytes = s.temp_bytes;
  BSA_HIP(hipcub::DeviceRadixSort::SortPairs(s.temp, bytes, s.keys_in, s.keys_out, s.vals_in, s.vals_out, (int)n, 0, 64,
                                             stream));
  return BSA_OK;
}

// ---- order of the output blocks for the tile kernel: super-tiles of tile x tile blocks of the block grid, the
// super-tiles of a batch entry row by row, the blocks of a super-tile row by row
__global__ __launch_bounds__(kThreads) void block_order_keys_kernel(const int64_t *__restrict__ coords, int64_t n,
                                                                    int64_t n_i, int64_t n_j, int tile,
                                                                    uint64_t *__restrict__ keys,
                                                                    int32_t *__restrict__ vals) {
  const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (e >= n) return;
  const int64_t b = coords[3 * e], i = coords[3 * e + 1], j = coords[3 * e + 2];
  keys[e] = (uint64_t)(((b * n_i + i / tile) * n_j + j / tile) * ((int64_t)tile * tile) + (i % tile) * tile + (j % tile));
  vals[e] = (int32_t)e;
}

__global__ __launch_bounds__(kThreads) void copy_i32_kernel(const int32_t *__restrict__ src, int64_t n,
                                                            int32_t *__restrict__ dst) {
  const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (e < n) dst[e] = src[e];
}

// ---- work table of the row kernel
struct TableShape {
  int64_t n_rows, rows_per_batch, n_entries, small, extra, heaviest;
  int parts_log2, pair_up, sweep;
};

__device__ inline int64_t chunk_of_row(int64_t row, const TableShape &t) {
  // chunk c holds small + 1 rows for c < extra and small rows after that
  const int64_t long_rows = t.extra * (t.small + 1);
  return row < long_rows ? row / (t.small + 1) : t.extra + (row - long_rows) / (t.small > 0 ? t.small : 1);
}

__global__ __launch_bounds__(kThreads) void work_table_keys_kernel(const int32_t *__restrict__ pair_offsets,
                                                                   const int32_t *__restrict__ row_offsets_o,
                                                                   TableShape t, uint64_t *__restrict__ keys,
                                                                   int32_t *__restrict__ vals) {
  const int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int64_t parts = (int64_t)1 << t.parts_log2;
  if (item >= t.n_rows * parts) return;
  const int64_t row = item >> t.parts_log2, part = item & (parts - 1);
  int64_t work = (int64_t)pair_offsets[row_offsets_o[row + 1]] - pair_offsets[row_offsets_o[row]];
  work = work < 0 ? 0 : (work > t.heaviest ? t.heaviest : work);  // a corrupt table must not leave its group
  const int64_t group = (chunk_of_row(row, t) * t.n_entries + row / t.rows_per_batch) * parts + part;
  keys[item] = (uint64_t)(group * (t.heaviest + 1) + (t.heaviest - work));
  vals[item] = (int32_t)item;
}

// first position in the sorted keys that is not below `key`
__device__ inline int64_t lower_bound(const uint64_t *keys, int64_t n, uint64_t key) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (keys[mid] < key) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(kThreads) void work_table_fill_kernel(int32_t *__restrict__ table, int64_t n) {
  const int64_t e = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (e < n) table[e] = -1;
}

__global__ __launch_bounds__(kThreads) void work_table_place_kernel(const uint64_t *__restrict__ keys,
                                                                    const int32_t *__restrict__ items, TableShape t,
                                                                    int32_t *__restrict__ table, int64_t table_len) {
  const int64_t parts = (int64_t)1 << t.parts_log2;
  const int64_t n = t.n_rows * parts;
  const int64_t p = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (p >= n) return;
  const int64_t span = t.heaviest + 1;
  const int64_t group = (int64_t)(keys[p] / (uint64_t)span);
  const int64_t start = lower_bound(keys, n, (uint64_t)(group * span));
  const int64_t rank = p - start;
  int64_t at = p;
  if (t.pair_up) {
    // within a group: longest, shortest, second longest, second shortest, ...
    const int64_t m = lower_bound(keys, n, (uint64_t)((group + 1) * span)) - start;
    at = start + (rank < (m + 1) / 2 ? 2 * rank : 2 * (m - 1 - rank) + 1);
  }
  const int64_t item = items[p];
  const int64_t row = item >> t.parts_log2;
  const int64_t chunk = chunk_of_row(row, t);
  const int64_t first_of_chunk = (chunk * t.small + (chunk < t.extra ? chunk : t.extra)) * parts;
  const int64_t slot = (at - first_of_chunk) * kXcds + chunk;
  int32_t code = (int32_t)item;
  if (t.sweep > 0 && ((rank / t.sweep) & 1)) code |= BSA_ROWS_DOWNWARD;
  if (slot >= 0 && slot < table_len) table[slot] = code;
}

}  // namespace

extern "C" size_t bsa_lut_order_workspace_bytes(int64_t n) { return n < 0 ? 0 : scratch_bytes(n); }

extern "C" int bsa_lut_block_order(const int64_t *layout_indices, int64_t n, int64_t n_rows, int64_t n_cols, int tile,
                                   int32_t *order, void *workspace, size_t workspace_bytes, bsa_stream_t stream) {
  const char *who = "bsa_lut_block_order";
  BSA_REQUIRE(n >= 0 && n < 0x7fffffffLL, "%s: bad number of blocks", who);
  BSA_REQUIRE(n_rows >= 0 && n_cols >= 0 && tile >= 1 && tile <= 1024, "%s: bad grid or tile size", who);
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(layout_indices && order && workspace, "%s: NULL pointer", who);
  BSA_REQUIRE(workspace_bytes >= scratch_bytes(n), "%s: workspace too small (%zu < %zu bytes)", who, workspace_bytes,
              scratch_bytes(n));
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "%s: workspace must be 256-byte aligned", who);
  hipStream_t s = bsa::as_stream(stream);
  const SortScratch sc = carve(workspace, n);
  const int64_t n_i = n_rows > 0 ? bsa::cdiv(n_rows, tile) : 1, n_j = n_cols > 0 ? bsa::cdiv(n_cols, tile) : 1;
  const unsigned grid = (unsigned)bsa::cdiv(n, kThreads);
  block_order_keys_kernel<<<grid, kThreads, 0, s>>>(layout_indices, n, n_i, n_j, tile, sc.keys_in, sc.vals_in);
  if (int rc = bsa::check_launch("block_order_keys_kernel")) return rc;
  if (int rc = sort_pairs(sc, n, s)) return rc;
  copy_i32_kernel<<<grid, kThreads, 0, s>>>(sc.vals_out, n, order);
  return bsa::check_launch("copy_i32_kernel");
}

extern "C" int bsa_lut_row_work_table(const int32_t *pair_offsets, const int32_t *row_offsets_o, int64_t n_rows,
                                      int64_t rows_per_batch, int parts_log2, int pair_up, int64_t max_work, int sweep,
                                      int32_t *table, int64_t table_len, void *workspace, size_t workspace_bytes,
                                      bsa_stream_t stream) {
  const char *who = "bsa_lut_row_work_table";
  BSA_REQUIRE(parts_log2 >= 0 && parts_log2 <= 3, "%s: parts_log2 must be 0..3 (got %d)", who, parts_log2);
  BSA_REQUIRE(n_rows >= 0 && (n_rows << parts_log2) < (int64_t)BSA_ROWS_DOWNWARD, "%s: bad number of block rows", who);
  BSA_REQUIRE(max_work >= 0 && max_work < ((int64_t)1 << 31), "%s: bad bound on the pairs of a row", who);
  BSA_REQUIRE(sweep >= 0, "%s: negative sweep", who);
  const int64_t parts = (int64_t)1 << parts_log2;
  const int64_t small = n_rows / kXcds, extra = n_rows % kXcds;
  const int64_t need = (small + (extra > 0 ? 1 : 0)) * parts * kXcds;
  BSA_REQUIRE(table_len == need, "%s: the table has %lld entries, %lld are needed", who, (long long)table_len,
              (long long)need);
  if (n_rows == 0) return BSA_OK;
  BSA_REQUIRE(pair_offsets && row_offsets_o && table && workspace, "%s: NULL pointer", who);
  const int64_t n = n_rows * parts;
  BSA_REQUIRE(workspace_bytes >= scratch_bytes(n), "%s: workspace too small (%zu < %zu bytes)", who, workspace_bytes,
              scratch_bytes(n));
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "%s: workspace must be 256-byte aligned", who);
  TableShape t;
  t.n_rows = n_rows;
  t.rows_per_batch = rows_per_batch > 0 ? rows_per_batch : 1;
  t.n_entries = n_rows / t.rows_per_batch + 1;
  t.small = small;
  t.extra = extra;
  t.heaviest = max_work;
  t.parts_log2 = parts_log2;
  t.pair_up = pair_up != 0;
  t.sweep = sweep;
  hipStream_t s = bsa::as_stream(stream);
  const SortScratch sc = carve(workspace, n);
  work_table_fill_kernel<<<(unsigned)bsa::cdiv(table_len, kThreads), kThreads, 0, s>>>(table, table_len);
  if (int rc = bsa::check_launch("work_table_fill_kernel")) return rc;
  const unsigned grid = (unsigned)bsa::cdiv(n, kThreads);
  work_table_keys_kernel<<<grid, kThreads, 0, s>>>(pair_offsets, row_offsets_o, t, sc.keys_in, sc.vals_in);
  if (int rc = bsa::check_launch("work_table_keys_kernel")) return rc;
  if (int rc = sort_pairs(sc, n, s)) return rc;
  work_table_place_kernel<<<grid, kThreads, 0, s>>>(sc.keys_out, sc.vals_out, t, table, table_len);
  return bsa::check_launch("work_table_place_kernel");
}
