// Layout -> lookup-table kernels (integer only, bit-exact).
//
// Everything derives from one primitive, an exclusive prefix sum over the
// flattened layout done in three launches (per-tile counts, a scan of the tile
// counts, a per-tile scan that writes results).  Tiles are 2048 entries; a
// layout of a million entries is 512 tiles.
#include "common.h"

#include <mutex>

namespace {

constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;

__device__ inline int to_count(uint8_t v) { return v != 0; }
__device__ inline int to_count(int32_t v) { return v; }

// Exclusive scan of one value per thread across a 256-thread block.
__device__ inline int block_exclusive_scan(int v, int &total) {
  __shared__ int wave_sums[kScanThreads / 64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int t = __shfl_up(incl, d);
    if (lane >= d) incl += t;
  }
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  int base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / 64; ++w) {
    int s = wave_sums[w];
    if (w < wave) base += s;
    tot += s;
  }
  __syncthreads();
  total = tot;
  return base + incl - v;
}

template <typename In>
__global__ __launch_bounds__(kScanThreads) void tile_counts_kernel(const In *__restrict__ in, int64_t n,
                                                                   int32_t *__restrict__ tile_counts) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int s = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t p = base + i;
    if (p < n) s += to_count(in[p]);
  }
  int total;
  block_exclusive_scan(s, total);
  if (threadIdx.x == 0) tile_counts[blockIdx.x] = total;
}

// One block: exclusive scan of the tile counts (int64 results), total -> stats[0],
// stats[1] = 0, and the closing entries of the optional outputs.
__global__ __launch_bounds__(kScanThreads) void scan_tiles_kernel(const int32_t *__restrict__ tile_counts,
                                                                  int64_t n_tiles,
                                                                  int64_t *__restrict__ tile_offsets,
                                                                  int64_t *__restrict__ stats,
                                                                  int32_t *__restrict__ last_i32) {
  int64_t carry = 0;
  for (int64_t start = 0; start < n_tiles; start += kScanThreads) {
    int64_t p = start + threadIdx.x;
    int v = p < n_tiles ? tile_counts[p] : 0;
    int total;
    int excl = block_exclusive_scan(v, total);
    if (p < n_tiles) tile_offsets[p] = carry + excl;
    carry += total;
  }
  if (threadIdx.x == 0) {
    stats[0] = carry;
    stats[1] = 0;
    if (last_i32) *last_i32 = (int32_t)carry;
  }
}

// Per tile: writes the reverse index and, when row_len > 0, the CSR offset of
// every row that starts inside the tile.
__global__ __launch_bounds__(kScanThreads) void write_packed_kernel(const uint8_t *__restrict__ layout, int64_t n,
                                                                    const int64_t *__restrict__ tile_offsets,
                                                                    int64_t row_len, int64_t *__restrict__ packed,
                                                                    int32_t *__restrict__ row_offsets) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int flags[kScanItems];
  int s = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t p = base + i;
    flags[i] = (p < n) ? to_count(layout[p]) : 0;
    s += flags[i];
  }
  int total;
  int64_t prefix = tile_offsets[blockIdx.x] + block_exclusive_scan(s, total);
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t p = base + i;
    if (p < n) {
      packed[p] = flags[i] ? prefix : (int64_t)-1;
      if (row_len > 0 && (p % row_len) == 0) row_offsets[p / row_len] = (int32_t)prefix;
      prefix += flags[i];
    }
  }
}

// Exclusive prefix of int32 counts (int32 out; the closing entry is written by scan_tiles_kernel).
__global__ __launch_bounds__(kScanThreads) void write_prefix_kernel(const int32_t *__restrict__ counts, int64_t n,
                                                                    const int64_t *__restrict__ tile_offsets,
                                                                    int32_t *__restrict__ out) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int vals[kScanItems];
  int s = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t p = base + i;
    vals[i] = (p < n) ? counts[p] : 0;
    s += vals[i];
  }
  int total;
  int64_t prefix = tile_offsets[blockIdx.x] + block_exclusive_scan(s, total);
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t p = base + i;
    if (p < n) {
      out[p] = (int32_t)prefix;
      prefix += vals[i];
    }
  }
}

__global__ void row_max_kernel(const int32_t *__restrict__ row_offsets, int64_t n_rows, int64_t *__restrict__ stats) {
  int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int c = 0;
  if (r < n_rows) c = row_offsets[r + 1] - row_offsets[r];
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) c = max(c, __shfl_xor(c, d));
  if ((threadIdx.x & 63) == 0 && c > 0)
    atomicMax(reinterpret_cast<unsigned long long *>(stats + 1), (unsigned long long)c);
}

__global__ void zero_stats_kernel(int64_t *stats, int32_t *row_offsets, int64_t n_rows_plus_1) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < 2) stats[i] = 0;
  if (row_offsets && i < n_rows_plus_1) row_offsets[i] = 0;
}

__global__ void nonzero_kernel(const int64_t *__restrict__ packed, int64_t n, int64_t R, int64_t C,
                               int64_t *__restrict__ coords) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  int64_t idx = packed[p];
  if (idx < 0) return;
  int64_t c = p % C;
  int64_t t = p / C;
  coords[idx * 3 + 0] = t / R;
  coords[idx * 3 + 1] = t % R;
  coords[idx * 3 + 2] = c;
}

__global__ void csr_indices_kernel(const int64_t *__restrict__ packed, int64_t n, int64_t C,
                                   int32_t *__restrict__ indices) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  int64_t idx = packed[p];
  if (idx >= 0) indices[idx] = (int32_t)(p % C);
}

__global__ void sorted_rows_kernel(const int32_t *__restrict__ row_offsets, int64_t n_rows, int64_t C,
                                   int64_t *__restrict__ sorted) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_rows * C) return;
  int64_t r = p / C, t = p % C;
  int64_t start = row_offsets[r], cnt = row_offsets[r + 1] - start;
  sorted[p] = t < cnt ? start + cnt - 1 - t : (int64_t)-1;
}

// lo[b,i,j] = any_k lx[b,i,k] & ly[b,k,j]; one thread per output entry, adjacent
// threads read adjacent bytes of ly.
__global__ void layout_matmul_kernel(const uint8_t *__restrict__ lx, const uint8_t *__restrict__ ly, int64_t B,
                                     int64_t R, int64_t K, int64_t C, uint8_t *__restrict__ lo) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= B * R * C) return;
  int64_t j = p % C;
  int64_t t = p / C;
  int64_t i = t % R, b = t / R;
  const uint8_t *xr = lx + (b * R + i) * K;
  const uint8_t *yc = ly + b * K * C + j;
  uint8_t any = 0;
  for (int64_t k = 0; k < K; ++k) any |= (uint8_t)((xr[k] != 0) & (yc[k * C] != 0));
  lo[p] = any;
}

// mask[(row)*W + w] bit t = pidx[row*K + 64w + t] >= 0
__global__ void row_masks_kernel(const int64_t *__restrict__ pidx, int64_t n_rows, int64_t K, int64_t W,
                                 uint64_t *__restrict__ mask) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n_rows * W) return;
  int64_t row = p / W, w = p % W;
  uint64_t m = 0;
  int64_t k0 = w * 64, k1 = min(K, k0 + 64);
  for (int64_t k = k0; k < k1; ++k)
    if (pidx[row * K + k] >= 0) m |= (uint64_t)1 << (k - k0);
  mask[p] = m;
}

// mask[(b*C + j)*W + w] bit t = pidx[(b*K + 64w + t)*C + j] >= 0; threads ordered (b, w, j).
__global__ void col_masks_kernel(const int64_t *__restrict__ pidx, int64_t B, int64_t K, int64_t C, int64_t W,
                                 uint64_t *__restrict__ mask) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= B * W * C) return;
  int64_t j = p % C;
  int64_t t = p / C;
  int64_t w = t % W, b = t / W;
  uint64_t m = 0;
  int64_t k0 = w * 64, k1 = min(K, k0 + 64);
  for (int64_t k = k0; k < k1; ++k)
    if (pidx[(b * K + k) * C + j] >= 0) m |= (uint64_t)1 << (k - k0);
  mask[(b * C + j) * W + w] = m;
}

__global__ void pair_counts_kernel(const int64_t *__restrict__ pidx_o, int64_t B, int64_t R, int64_t C, int64_t W,
                                   const uint64_t *__restrict__ mask_x, const uint64_t *__restrict__ mask_y,
                                   int32_t *__restrict__ counts) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= B * R * C) return;
  int c = 0;
  if (pidx_o[p] >= 0) {
    int64_t j = p % C;
    int64_t t = p / C;
    int64_t b = t / R;
    const uint64_t *mx = mask_x + t * W;
    const uint64_t *my = mask_y + (b * C + j) * W;
    for (int64_t w = 0; w < W; ++w) c += __popcll(mx[w] & my[w]);
  }
  counts[p] = c;
}

__global__ void pairs_kernel(const int64_t *__restrict__ pidx_x, const int64_t *__restrict__ pidx_y,
                             const int64_t *__restrict__ pidx_o, int64_t B, int64_t R, int64_t K, int64_t C,
                             int64_t W, const uint64_t *__restrict__ mask_x, const uint64_t *__restrict__ mask_y,
                             const int32_t *__restrict__ pos_offsets, int64_t nnz_o,
                             int32_t *__restrict__ pair_offsets, int32_t *__restrict__ pairs) {
  int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n = B * R * C;
  if (p == 0) pair_offsets[nnz_o] = pos_offsets[n];
  if (p >= n) return;
  int64_t o = pidx_o[p];
  if (o < 0 || o >= nnz_o) return;
  int64_t j = p % C;
  int64_t t = p / C;  // b*R + i
  int64_t b = t / R;
  int32_t off = pos_offsets[p];
  pair_offsets[o] = off;
  const uint64_t *mx = mask_x + t * W;
  const uint64_t *my = mask_y + (b * C + j) * W;
  for (int64_t w = 0; w < W; ++w) {
    uint64_t m = mx[w] & my[w];
    while (m) {
      int bit = __ffsll((unsigned long long)m) - 1;
      m &= m - 1;
      int64_t k = w * 64 + bit;
      pairs[2 * (int64_t)off + 0] = (int32_t)pidx_x[t * K + k];
      pairs[2 * (int64_t)off + 1] = (int32_t)pidx_y[(b * K + k) * C + j];
      ++off;
    }
  }
}

struct ScanWorkspace {
  int32_t *tile_counts;
  int64_t *tile_offsets;
  int32_t *counts;  // per-position pair counts (contraction builder only)
};

size_t scan_workspace_bytes(int64_t n) {
  int64_t tiles = bsa::cdiv(n > 0 ? n : 1, kScanTile);
  size_t a = ((size_t)tiles * 4 + 255) / 256 * 256;
  size_t b = ((size_t)tiles * 8 + 255) / 256 * 256;
  size_t c = ((size_t)(n > 0 ? n : 1) * 4 + 255) / 256 * 256;
  return a + b + c;
}

ScanWorkspace carve(void *workspace, int64_t n) {
  int64_t tiles = bsa::cdiv(n > 0 ? n : 1, kScanTile);
  size_t a = ((size_t)tiles * 4 + 255) / 256 * 256;
  size_t b = ((size_t)tiles * 8 + 255) / 256 * 256;
  char *base = static_cast<char *>(workspace);
  ScanWorkspace w;
  w.tile_counts = reinterpret_cast<int32_t *>(base);
  w.tile_offsets = reinterpret_cast<int64_t *>(base + a);
  w.counts = reinterpret_cast<int32_t *>(base + a + b);
  return w;
}

int fetch_stats(const int64_t *stats_dev, int64_t *stats_host, hipStream_t s) {
  if (!stats_host) return BSA_OK;
  BSA_HIP(hipMemcpyAsync(stats_host, stats_dev, 2 * sizeof(int64_t), hipMemcpyDeviceToHost, s));
  BSA_HIP(hipStreamSynchronize(s));
  return BSA_OK;
}

inline unsigned grid_for(int64_t n, int threads) { return (unsigned)bsa::cdiv(n, threads); }

}  // namespace

extern "C" size_t bsa_lut_workspace_bytes(int64_t n) { return scan_workspace_bytes(n); }

namespace {

// The launches of the scan; tile_counts (int32) and tile_offsets (int64) hold one entry per tile of kScanTile
// layout entries and are written before they are read.
int lut_packed_launch(const char *who, const uint8_t *layout, int64_t n, int64_t row_len, int64_t *packed,
                      int32_t *row_offsets, int64_t *stats_dev, int64_t *stats_host, int32_t *tile_counts,
                      int64_t *tile_offsets, hipStream_t s) {
  BSA_REQUIRE(n >= 0 && row_len >= 0, "%s: negative size", who);
  BSA_REQUIRE(stats_dev != nullptr, "%s: stats_dev is NULL", who);
  BSA_REQUIRE(row_len == 0 || row_offsets != nullptr, "%s: row_len given without row_offsets", who);
  BSA_REQUIRE(row_len == 0 || n % row_len == 0, "%s: n is not a multiple of row_len", who);
  if (n / kScanTile >= 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "%s: layout too large", who);
  if (n == 0) {
    // row_len > 0 with n == 0 still has the leading 0 (n_rows is 0 then).
    zero_stats_kernel<<<1, 64, 0, s>>>(stats_dev, row_len > 0 ? row_offsets : nullptr, 1);
    if (int rc = bsa::check_launch("zero_stats_kernel")) return rc;
    return fetch_stats(stats_dev, stats_host, s);
  }
  BSA_REQUIRE(layout && packed, "%s: NULL layout or output", who);
  BSA_REQUIRE(tile_counts && tile_offsets, "%s: no workspace", who);
  const int64_t tiles = bsa::cdiv(n, kScanTile);
  const int64_t n_rows = row_len > 0 ? n / row_len : 0;
  tile_counts_kernel<uint8_t><<<(unsigned)tiles, kScanThreads, 0, s>>>(layout, n, tile_counts);
  scan_tiles_kernel<<<1, kScanThreads, 0, s>>>(tile_counts, tiles, tile_offsets, stats_dev,
                                               row_len > 0 ? row_offsets + n_rows : nullptr);
  write_packed_kernel<<<(unsigned)tiles, kScanThreads, 0, s>>>(layout, n, tile_offsets, row_len, packed, row_offsets);
  if (row_len > 0) row_max_kernel<<<grid_for(n_rows, 256), 256, 0, s>>>(row_offsets, n_rows, stats_dev);
  if (int rc = bsa::check_launch(who)) return rc;
  return fetch_stats(stats_dev, stats_host, s);
}

}  // namespace

extern "C" int bsa_lut_packed(const uint8_t *layout, int64_t n, int64_t row_len, int64_t *packed,
                              int32_t *row_offsets, int64_t *stats_dev, int64_t *stats_host, void *workspace,
                              size_t workspace_bytes, bsa_stream_t stream) {
  BSA_REQUIRE(n <= 0 || (workspace && workspace_bytes >= scan_workspace_bytes(n)),
              "bsa_lut_packed: workspace too small");
  ScanWorkspace w = carve(workspace, n);
  return lut_packed_launch("bsa_lut_packed", layout, n, row_len, packed, row_offsets, stats_dev, stats_host,
                           n > 0 ? w.tile_counts : nullptr, n > 0 ? w.tile_offsets : nullptr, bsa::as_stream(stream));
}

// ---------------------------------------------------------------------------------------------------
// bsa_lut_packed_static: the scan of bsa_lut_packed with its tile counts and tile offsets in a file-scope
// device array instead of a caller-provided workspace, for callers that cannot allocate.
namespace {

constexpr int64_t kStaticMaxEntries = (int64_t)1 << 24;                  // layout entries per call
constexpr int64_t kStaticMaxTiles = kStaticMaxEntries / kScanTile;       // 8192
constexpr size_t kStaticScratchBytes = (size_t)kStaticMaxTiles * (4 + 8);  // 96 KiB per device

}  // namespace

// Every device the library runs on holds its own copy of this array, at its own address.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex static_scratch_mutex;
void *static_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (looked up once per device; the host-side name
// of the array is not an address a kernel can use).
int static_scratch(void **out) {
  int dev = -1;
  BSA_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return bsa::fail(BSA_ELIMIT, "bsa_lut_packed_static: device %d out of range", dev);
  std::lock_guard<std::mutex> lock(static_scratch_mutex);
  if (!static_scratch_ptr[dev]) {
    void *p = nullptr;
    BSA_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return bsa::fail(BSA_ELAUNCH, "bsa_lut_packed_static: no device address for the scratch array");
    static_scratch_ptr[dev] = p;
  }
  *out = static_scratch_ptr[dev];
  return BSA_OK;
}

}  // namespace

extern "C" int64_t bsa_lut_packed_static_max_entries(void) { return kStaticMaxEntries; }

extern "C" int bsa_lut_packed_static(const uint8_t *layout, int64_t n, int64_t row_len, int64_t *packed,
                                     int32_t *row_offsets, int64_t *stats_dev, bsa_stream_t stream) {
  BSA_REQUIRE(n >= 0 && row_len >= 0, "bsa_lut_packed_static: negative size");
  if (n > kStaticMaxEntries)
    return bsa::fail(BSA_ELIMIT, "bsa_lut_packed_static: %lld layout entries exceed the static scratch (at most %lld)",
                     (long long)n, (long long)kStaticMaxEntries);
  void *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // Same launches as bsa_lut_packed; every tile count and tile offset that is read is written first by this
  // call, so what an earlier call left in the array does not matter.
  int32_t *tile_counts = static_cast<int32_t *>(ws);
  int64_t *tile_offsets = reinterpret_cast<int64_t *>(static_cast<char *>(ws) + kStaticMaxTiles * 4);
  return lut_packed_launch("bsa_lut_packed_static", layout, n, row_len, packed, row_offsets, stats_dev, nullptr,
                           tile_counts, tile_offsets, bsa::as_stream(stream));
}

extern "C" int bsa_lut_nonzero(const int64_t *packed, int64_t B, int64_t R, int64_t C, int64_t *coords,
                               bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && C >= 0, "bsa_lut_nonzero: negative size");
  const int64_t n = B * R * C;
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(packed && coords, "bsa_lut_nonzero: NULL pointer");
  nonzero_kernel<<<grid_for(n, 256), 256, 0, bsa::as_stream(stream)>>>(packed, n, R, C, coords);
  return bsa::check_launch("nonzero_kernel");
}

extern "C" int bsa_lut_csr_indices(const int64_t *packed, int64_t n, int64_t C, int32_t *indices,
                                   bsa_stream_t stream) {
  BSA_REQUIRE(n >= 0 && C >= 0, "bsa_lut_csr_indices: negative size");
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(packed && indices && C > 0, "bsa_lut_csr_indices: NULL pointer or C == 0");
  csr_indices_kernel<<<grid_for(n, 256), 256, 0, bsa::as_stream(stream)>>>(packed, n, C, indices);
  return bsa::check_launch("csr_indices_kernel");
}

// ---- lists over pairs of neighbouring rows (the attention forward's groups of two query blocks)
// the union of rows 2 g and 2 g + 1 of a layout of 0/1 bytes [B, R, C], as bytes [B, ceil(R / 2), C]
__global__ __launch_bounds__(256) void pair_union_kernel(const uint8_t *__restrict__ layout, int64_t B, int64_t R,
                                                         int64_t C, uint8_t *__restrict__ uni) {
  const int64_t G = (R + 1) / 2;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= B * G * C) return;
  const int64_t c = e % C, g = (e / C) % G, b = e / (C * G);
  const uint8_t first = layout[(b * R + 2 * g) * C + c];
  const uint8_t second = 2 * g + 1 < R ? layout[(b * R + 2 * g + 1) * C + c] : (uint8_t)0;
  uni[e] = (first | second) ? 1 : 0;
}

// entries[p] = column | first row active << 28 | second row active << 29 for the p-th active position of the union
__global__ __launch_bounds__(256) void pair_entries_kernel(const uint8_t *__restrict__ layout,
                                                           const int64_t *__restrict__ union_packed, int64_t B,
                                                           int64_t R, int64_t C, int32_t *__restrict__ entries) {
  const int64_t G = (R + 1) / 2;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= B * G * C) return;
  const int64_t p = union_packed[e];
  if (p < 0) return;
  const int64_t c = e % C, g = (e / C) % G, b = e / (C * G);
  const int32_t first = layout[(b * R + 2 * g) * C + c] ? 1 : 0;
  const int32_t second = (2 * g + 1 < R && layout[(b * R + 2 * g + 1) * C + c]) ? 1 : 0;
  entries[p] = (int32_t)c | (first << 28) | (second << 29);
}

extern "C" int bsa_lut_pair_union(const uint8_t *layout, int64_t B, int64_t R, int64_t C, uint8_t *uni,
                                  bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && C >= 0, "bsa_lut_pair_union: negative size");
  const int64_t n = B * ((R + 1) / 2) * C;
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(layout && uni, "bsa_lut_pair_union: NULL pointer");
  pair_union_kernel<<<grid_for(n, 256), 256, 0, bsa::as_stream(stream)>>>(layout, B, R, C, uni);
  return bsa::check_launch("pair_union_kernel");
}

extern "C" int bsa_lut_pair_entries(const uint8_t *layout, const int64_t *union_packed, int64_t B, int64_t R,
                                    int64_t C, int32_t *entries, bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && C >= 0, "bsa_lut_pair_entries: negative size");
  BSA_REQUIRE(C < (1 << 28), "bsa_lut_pair_entries: too many columns for an entry");
  const int64_t n = B * ((R + 1) / 2) * C;
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(layout && union_packed && entries, "bsa_lut_pair_entries: NULL pointer");
  pair_entries_kernel<<<grid_for(n, 256), 256, 0, bsa::as_stream(stream)>>>(layout, union_packed, B, R, C, entries);
  return bsa::check_launch("pair_entries_kernel");
}

extern "C" int bsa_lut_sorted_rows(const int32_t *row_offsets, int64_t n_rows, int64_t C, int64_t *sorted,
                                   bsa_stream_t stream) {
  BSA_REQUIRE(n_rows >= 0 && C >= 0, "bsa_lut_sorted_rows: negative size");
  if (n_rows * C == 0) return BSA_OK;
  BSA_REQUIRE(row_offsets && sorted, "bsa_lut_sorted_rows: NULL pointer");
  sorted_rows_kernel<<<grid_for(n_rows * C, 256), 256, 0, bsa::as_stream(stream)>>>(row_offsets, n_rows, C, sorted);
  return bsa::check_launch("sorted_rows_kernel");
}

extern "C" int bsa_layout_matmul(const uint8_t *lx, const uint8_t *ly, int64_t B, int64_t R, int64_t K, int64_t C,
                                 uint8_t *lo, bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && K >= 0 && C >= 0, "bsa_layout_matmul: negative size");
  const int64_t n = B * R * C;
  if (n == 0) return BSA_OK;
  BSA_REQUIRE(lo && (K == 0 || (lx && ly)), "bsa_layout_matmul: NULL pointer");
  layout_matmul_kernel<<<grid_for(n, 256), 256, 0, bsa::as_stream(stream)>>>(lx, ly, B, R, K, C, lo);
  return bsa::check_launch("layout_matmul_kernel");
}

extern "C" int bsa_lut_contraction_offsets(const int64_t *pidx_x, const int64_t *pidx_y, const int64_t *pidx_o,
                                           int64_t B, int64_t R, int64_t K, int64_t C, uint64_t *mask_x,
                                           uint64_t *mask_y, int32_t *pos_offsets, int64_t *stats_dev,
                                           int64_t *stats_host, void *workspace, size_t workspace_bytes,
                                           bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && K >= 0 && C >= 0, "bsa_lut_contraction_offsets: negative size");
  BSA_REQUIRE(stats_dev && pos_offsets, "bsa_lut_contraction_offsets: NULL output");
  hipStream_t s = bsa::as_stream(stream);
  const int64_t n = B * R * C;
  const int64_t W = bsa::cdiv(K, 64);
  if (n == 0) {
    zero_stats_kernel<<<1, 64, 0, s>>>(stats_dev, pos_offsets, 1);
    if (int rc = bsa::check_launch("zero_stats_kernel")) return rc;
    return fetch_stats(stats_dev, stats_host, s);
  }
  BSA_REQUIRE(pidx_o && (K == 0 || (pidx_x && pidx_y && mask_x && mask_y)),
              "bsa_lut_contraction_offsets: NULL pointer");
  BSA_REQUIRE(workspace && workspace_bytes >= scan_workspace_bytes(n),
              "bsa_lut_contraction_offsets: workspace too small");
  if (n / kScanTile >= 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_lut_contraction_offsets: layout too large");
  ScanWorkspace w = carve(workspace, n);
  if (W > 0) {
    row_masks_kernel<<<grid_for(B * R * W, 256), 256, 0, s>>>(pidx_x, B * R, K, W, mask_x);
    col_masks_kernel<<<grid_for(B * W * C, 256), 256, 0, s>>>(pidx_y, B, K, C, W, mask_y);
  }
  pair_counts_kernel<<<grid_for(n, 256), 256, 0, s>>>(pidx_o, B, R, C, W, mask_x, mask_y, w.counts);
  const int64_t tiles = bsa::cdiv(n, kScanTile);
  tile_counts_kernel<int32_t><<<(unsigned)tiles, kScanThreads, 0, s>>>(w.counts, n, w.tile_counts);
  scan_tiles_kernel<<<1, kScanThreads, 0, s>>>(w.tile_counts, tiles, w.tile_offsets, stats_dev, pos_offsets + n);
  write_prefix_kernel<<<(unsigned)tiles, kScanThreads, 0, s>>>(w.counts, n, w.tile_offsets, pos_offsets);
  if (int rc = bsa::check_launch("bsa_lut_contraction_offsets")) return rc;
  return fetch_stats(stats_dev, stats_host, s);
}

extern "C" int bsa_lut_contraction_pairs(const int64_t *pidx_x, const int64_t *pidx_y, const int64_t *pidx_o,
                                         int64_t B, int64_t R, int64_t K, int64_t C, const uint64_t *mask_x,
                                         const uint64_t *mask_y, const int32_t *pos_offsets, int64_t nnz_o,
                                         int32_t *pair_offsets, int32_t *pairs, bsa_stream_t stream) {
  BSA_REQUIRE(B >= 0 && R >= 0 && K >= 0 && C >= 0 && nnz_o >= 0, "bsa_lut_contraction_pairs: negative size");
  BSA_REQUIRE(pair_offsets && pos_offsets, "bsa_lut_contraction_pairs: NULL pointer");
  const int64_t n = B * R * C;
  const int64_t W = bsa::cdiv(K, 64);
  // at least one thread so that the closing offset is written
  const int64_t threads = n > 0 ? n : 1;
  pairs_kernel<<<grid_for(threads, 256), 256, 0, bsa::as_stream(stream)>>>(
      pidx_x, pidx_y, pidx_o, B, R, K, C, W, mask_x, mask_y, pos_offsets, nnz_o, pair_offsets, pairs);
  return bsa::check_launch("pairs_kernel");
}
