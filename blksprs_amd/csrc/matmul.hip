// Block-sparse GEMM: out[n] = sum over the contraction list of block n of x[px] @ y[py].
//
// One wavefront owns one TILE x TILE tile of one output block (TILE = min(sbs, 64))
// and walks that block's list of (x block, y block) pairs in ascending k, so only
// non-zero K-blocks are touched and the fp32 accumulation order is fixed.  Four
// waves (four neighbouring tiles) share a workgroup but never synchronise: each
// has a private 16 KiB LDS region.
//
// Data path per K-chunk (64 k for 16-bit types, 32 k for fp32):
//   global --16 B per lane, consecutive lanes = consecutive bytes--> VGPRs
//          --ds_write_b128--> LDS --> MFMA operand fragments --> v_mfma_f32_32x32x*.
// The loads of chunk t+1 are issued before the MFMAs of chunk t.
//
// An operand whose k index is contiguous in memory (x, or y read transposed) is
// kept row-major in LDS with the 16-byte chunks of a row XOR-swizzled, and a
// fragment is one ds_read_b128.  An operand whose k index is strided (y, or x read
// transposed) cannot be fed to the matrix core as stored, because a lane needs 8
// consecutive k of one column: for 16-bit types two k rows are interleaved in
// registers (v_perm_b32) before the LDS write, so LDS holds (k, k+1) pairs per
// column and a fragment is four conflict-free ds_read_b32; fp32 needs no packing.
//
// The product is formed transposed (y fragments as the A operand, x fragments as
// B), which leaves 4 consecutive output columns of one row in each lane; the tile
// is rounded to the output type, staged through LDS and written with 16-byte
// stores that cover whole rows.
//
// sbs == 16 has kernels of its own (16 x 16 x 16 products for 16-bit elements, FMAs
// for fp32): at 13 flop/byte it is a gather problem, not a matrix-core problem.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <type_traits>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
// native vector (not HIP's uint4 struct): arrays of it are always promoted to registers
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct Bf16Traits {
  static constexpr int kElem = 2;
  using store_t = uint16_t;
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  // round to nearest even, NaN kept quiet (the hardware conversion of gfx950)
  __device__ static uint16_t round(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
  __device__ static float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
};

struct F16Traits {
  static constexpr int kElem = 2;
  using store_t = uint16_t;
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
  __device__ static uint16_t round(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
  __device__ static float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
};

struct F32Traits {
  static constexpr int kElem = 4;
  using store_t = float;
  // by-value helper: __builtin_bit_cast applied directly to a vector component reads component 0
  __device__ static float as_float(uint32_t v) { return __builtin_bit_cast(float, v); }
  // one fragment = 4 floats = 4 rank-2 updates
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(as_float(a[0]), as_float(b[0]), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(as_float(a[1]), as_float(b[1]), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(as_float(a[2]), as_float(b[2]), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(as_float(a[3]), as_float(b[3]), c, 0, 0, 0);
    return c;
  }
  __device__ static float round(float v) { return v; }
  __device__ static float widen(float v) { return v; }
};

// Geometry of one operand chunk in LDS (TILE rows of the non-contracted index, KC values of k).
template <typename Tr, int TILE>
struct Geom {
  static constexpr int ES = Tr::kElem;
  static constexpr int KC = (ES == 2) ? TILE : 32;       // k per chunk
  static constexpr int STEPS = (ES == 2) ? KC / 16 : KC / 8;  // fragments along k per chunk
  static constexpr int NB = TILE / 32;                    // 32-wide MFMA blocks per side
  static constexpr int REGION = TILE * KC * ES;           // bytes of one operand chunk
  // k-contiguous staging
  static constexpr int CPR = KC * ES / 16;                // 16-byte chunks per row
  static constexpr int RPL = (CPR >= 8) ? 1 : 8 / CPR;    // rows per 128-byte LDS line
  static constexpr int KCONT_LOADS = TILE * CPR / 64;     // uint4 per lane
  // k-strided staging
  static constexpr int KSTR_LOADS = (ES == 2) ? (KC / 2) * (TILE / 8) * 2 / 64 : KC * (TILE / 4) / 64;
  static constexpr int LOADS = KCONT_LOADS > KSTR_LOADS ? KCONT_LOADS : KSTR_LOADS;
  // output staging
  static constexpr int OCPR = TILE * ES / 16;
  static constexpr int OUT_STORES = TILE * OCPR / 64;
  static constexpr int OUT_BYTES = TILE * TILE * ES;
  static constexpr int WAVE_LDS = (2 * REGION > OUT_BYTES) ? 2 * REGION : OUT_BYTES;
};

template <int CPR, int RPL>
__device__ inline int swizzle(int row, int chunk) {
  return chunk ^ ((row / RPL) & (CPR - 1));
}

// Dword offset of column c inside pair row kp of the (k, k+1)-packed layout of a k-strided operand.
// Columns are kept in quads (one ds_write_b128 each).  Quad q = 2a + h is placed so that (i) the eight
// lanes that write the even (or the odd) quads of consecutive column octets hit eight different quad
// banks and (ii) the 32 lanes that read 32 consecutive columns of one pair row do too.
template <int TILE>
__device__ inline int pair_col_offset(int kp, int c) {
  const int q = c >> 2, a = q >> 1, h = q & 1;
  int pos;
  if constexpr (TILE == 64)
    pos = ((a + 4 * h) & 7) + 8 * h;
  else
    pos = a + 4 * (h ^ (kp & 1));
  return 4 * pos + (c & 3);
}

// ---- global -> registers -------------------------------------------------

// k contiguous: element (row, k) at base[row * ld + k]
template <typename G>
__device__ inline void load_kcont(u32x4 (&r)[G::LOADS], const char *base, uint32_t ld_bytes, int lane) {
#pragma unroll
  for (int i = 0; i < G::KCONT_LOADS; ++i) {
    const int q = i * 64 + lane;
    const int row = q / G::CPR, c = q % G::CPR;
    r[i] = *reinterpret_cast<const u32x4 *>(base + (uint32_t)(row * ld_bytes + c * 16));
  }
}

// k strided: element (row, k) at base[k * ld + row]
template <typename G, int TILE>
__device__ inline void load_kstr(u32x4 (&r)[G::LOADS], const char *base, uint32_t ld_bytes, int lane) {
  if constexpr (G::ES == 2) {
#pragma unroll
    for (int i = 0; i < G::KSTR_LOADS / 2; ++i) {
      const int q = i * 64 + lane;
      const int ro = q % (TILE / 8), kp = q / (TILE / 8);
      r[2 * i] = *reinterpret_cast<const u32x4 *>(base + (uint32_t)((2 * kp) * ld_bytes + ro * 16));
      r[2 * i + 1] = *reinterpret_cast<const u32x4 *>(base + (uint32_t)((2 * kp + 1) * ld_bytes + ro * 16));
    }
  } else {
#pragma unroll
    for (int i = 0; i < G::KSTR_LOADS; ++i) {
      const int q = i * 64 + lane;
      const int rc = q % (TILE / 4), k = q / (TILE / 4);
      r[i] = *reinterpret_cast<const u32x4 *>(base + (uint32_t)(k * ld_bytes + rc * 16));
    }
  }
}

// ---- registers -> LDS ----------------------------------------------------

template <typename G>
__device__ inline void stage_kcont(const u32x4 (&r)[G::LOADS], char *lds, int lane) {
#pragma unroll
  for (int i = 0; i < G::KCONT_LOADS; ++i) {
    const int q = i * 64 + lane;
    const int row = q / G::CPR, c = q % G::CPR;
    *reinterpret_cast<u32x4 *>(lds + row * (G::CPR * 16) + swizzle<G::CPR, G::RPL>(row, c) * 16) = r[i];
  }
}

template <typename G, int TILE>
__device__ inline void stage_kstr(const u32x4 (&r)[G::LOADS], char *lds, int lane) {
  if constexpr (G::ES == 2) {
#pragma unroll
    for (int i = 0; i < G::KSTR_LOADS / 2; ++i) {
      const int q = i * 64 + lane;
      const int ro = q % (TILE / 8), kp = q / (TILE / 8);
      const u32x4 e = r[2 * i], o = r[2 * i + 1];  // rows 2kp and 2kp+1, 8 columns each
      // dword for column c = (even-row value, odd-row value)
      u32x4 lo, hi;
      lo.x = __builtin_amdgcn_perm(o.x, e.x, 0x05040100u);
      lo.y = __builtin_amdgcn_perm(o.x, e.x, 0x07060302u);
      lo.z = __builtin_amdgcn_perm(o.y, e.y, 0x05040100u);
      lo.w = __builtin_amdgcn_perm(o.y, e.y, 0x07060302u);
      hi.x = __builtin_amdgcn_perm(o.z, e.z, 0x05040100u);
      hi.y = __builtin_amdgcn_perm(o.z, e.z, 0x07060302u);
      hi.z = __builtin_amdgcn_perm(o.w, e.w, 0x05040100u);
      hi.w = __builtin_amdgcn_perm(o.w, e.w, 0x07060302u);
      uint32_t *row = reinterpret_cast<uint32_t *>(lds) + kp * TILE;
      *reinterpret_cast<u32x4 *>(row + pair_col_offset<TILE>(kp, ro * 8)) = lo;
      *reinterpret_cast<u32x4 *>(row + pair_col_offset<TILE>(kp, ro * 8 + 4)) = hi;
    }
  } else {
#pragma unroll
    for (int i = 0; i < G::KSTR_LOADS; ++i) {
      const int q = i * 64 + lane;
      const int rc = q % (TILE / 4), k = q / (TILE / 4);
      *reinterpret_cast<u32x4 *>(reinterpret_cast<uint32_t *>(lds) + k * TILE + rc * 4) = r[i];
    }
  }
}

// ---- LDS -> MFMA fragment ------------------------------------------------
// fragment (block mb, step s) of lane (row = 32 mb + lane % 32, kg = lane / 32)

template <typename G>
__device__ inline u32x4 frag_kcont(const char *lds, int mb, int s, int lane) {
  const int row = 32 * mb + (lane & 31), kg = lane >> 5;
  return *reinterpret_cast<const u32x4 *>(lds + row * (G::CPR * 16) + swizzle<G::CPR, G::RPL>(row, 2 * s + kg) * 16);
}

template <typename G, int TILE>
__device__ inline u32x4 frag_kstr(const char *lds, int mb, int s, int lane) {
  const int row = 32 * mb + (lane & 31), kg = lane >> 5;
  // 16-bit: (k,k+1) pair rows 8s + 4kg + t; fp32: k rows 8s + 4kg + t
  const uint32_t *p = reinterpret_cast<const uint32_t *>(lds) + (8 * s + 4 * kg) * TILE;
  u32x4 v;
  if constexpr (G::ES == 2) {
    v[0] = p[pair_col_offset<TILE>(0, row)];
    v[1] = p[TILE + pair_col_offset<TILE>(1, row)];
    v[2] = p[2 * TILE + pair_col_offset<TILE>(0, row)];
    v[3] = p[3 * TILE + pair_col_offset<TILE>(1, row)];
  } else {
    v[0] = p[row];
    v[1] = p[TILE + row];
    v[2] = p[2 * TILE + row];
    v[3] = p[3 * TILE + row];
  }
  return v;
}

template <typename Tr, int TILE, bool XT, bool YT>
__global__ __launch_bounds__(256, 2) void matmul_mfma_kernel(const char *__restrict__ x, const char *__restrict__ y,
                                                             char *__restrict__ out,
                                                             const int32_t *__restrict__ pair_offsets,
                                                             const int32_t *__restrict__ pairs,
                                                             const int32_t *__restrict__ block_order,
                                                             int64_t n_tiles, int sbs, int side_log2, int64_t nnz_x,
                                                             int64_t nnz_y) {
  using G = Geom<Tr, TILE>;
  constexpr int ES = G::ES;
  __shared__ __attribute__((aligned(16))) char smem[4 * G::WAVE_LDS];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give XCD c the c-th contiguous
  // eighth of the (ordered) work list, so that the tiles in flight on one L2 are neighbours in the list.
  const int64_t per_xcd = gridDim.x >> 3;
  const int64_t group = (int64_t)(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int64_t item = group * 4 + wave;
  if (item >= n_tiles) return;
  int64_t tile = item;
  if (block_order) {
    const int64_t per_block = (int64_t)1 << (2 * side_log2);
    tile = (int64_t)__builtin_amdgcn_readfirstlane(block_order[item >> (2 * side_log2)]) * per_block +
           (item & (per_block - 1));
  }
  char *lds_x = smem + wave * G::WAVE_LDS;
  char *lds_y = lds_x + G::REGION;

  const int side_mask = (1 << side_log2) - 1;
  const int64_t n = tile >> (2 * side_log2);
  const int ti = (int)(tile >> side_log2) & side_mask;
  const int tj = (int)tile & side_mask;
  const int64_t block_bytes = (int64_t)sbs * sbs * ES;
  const uint32_t ld_bytes = (uint32_t)sbs * ES;
  const int n_chunks = sbs / G::KC;  // K-chunks per pair

  const int p_begin = __builtin_amdgcn_readfirstlane(pair_offsets[n]);
  const int p_end = __builtin_amdgcn_readfirstlane(pair_offsets[n + 1]);
  const int n_iter = (p_end - p_begin) * n_chunks;

  f32x16 acc[G::NB][G::NB];  // [block along j][block along i]
#pragma unroll
  for (int a = 0; a < G::NB; ++a)
#pragma unroll
    for (int b = 0; b < G::NB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  u32x4 rx[G::LOADS], ry[G::LOADS];

  // 64 entries of this block's pair list at a time, one per lane (a dependent index load per K-chunk would
  // put a full memory latency on the critical path of every iteration)
  int win_base = p_begin, win_px = 0, win_py = 0;
#define BSA_LOAD_WINDOW()                                                            \
  do {                                                                               \
    const int t_ = win_base + lane;                                                  \
    win_px = win_py = 0;                                                             \
    if (t_ < p_end) {                                                                \
      const int2 v_ = *reinterpret_cast<const int2 *>(pairs + 2 * (int64_t)t_);      \
      win_px = v_.x;                                                                 \
      win_py = v_.y;                                                                 \
    }                                                                                \
  } while (0)
  BSA_LOAD_WINDOW();

  // Issues the global loads of iteration `it` (pair it / n_chunks, K-chunk it % n_chunks) into rx / ry.
#define BSA_FETCH(it_)                                                                                           \
  do {                                                                                                           \
    const int p_ = p_begin + (it_) / n_chunks;                                                                   \
    const int kc_ = (it_) % n_chunks;                                                                            \
    /* the pair indices come from a 64-entry register window, not from memory: no load latency here */          \
    if (p_ - win_base >= 64) {                                                                                   \
      win_base += 64;                                                                                            \
      BSA_LOAD_WINDOW();                                                                                         \
    }                                                                                                            \
    const int sel_ = __builtin_amdgcn_readfirstlane(p_ - win_base);                                              \
    int64_t px_ = __builtin_amdgcn_readlane(win_px, sel_);                                                       \
    int64_t py_ = __builtin_amdgcn_readlane(win_py, sel_);                                                       \
    /* a corrupt list must not turn into a wild read */                                                         \
    px_ = (px_ < 0 || px_ >= nnz_x) ? 0 : px_;                                                                   \
    py_ = (py_ < 0 || py_ >= nnz_y) ? 0 : py_;                                                                   \
    const char *xb_ = x + px_ * block_bytes;                                                                     \
    const char *yb_ = y + py_ * block_bytes;                                                                     \
    /* x tile: rows i = ti*TILE.., k = kc*KC..;  y tile: k rows, columns j = tj*TILE.. */                        \
    if constexpr (!XT)                                                                                           \
      load_kcont<G>(rx, xb_ + (int64_t)ti * TILE * (int64_t)ld_bytes + (int64_t)kc_ * G::KC * ES, ld_bytes, lane);        \
    else /* block holds x^T: element (i, k) at blk[k][i] */                                                      \
      load_kstr<G, TILE>(rx, xb_ + (int64_t)kc_ * G::KC * (int64_t)ld_bytes + (int64_t)ti * TILE * ES, ld_bytes, lane);   \
    if constexpr (!YT)                                                                                           \
      load_kstr<G, TILE>(ry, yb_ + (int64_t)kc_ * G::KC * (int64_t)ld_bytes + (int64_t)tj * TILE * ES, ld_bytes, lane);   \
    else /* block holds y^T: element (k, j) at blk[j][k] */                                                      \
      load_kcont<G>(ry, yb_ + (int64_t)tj * TILE * (int64_t)ld_bytes + (int64_t)kc_ * G::KC * ES, ld_bytes, lane);        \
  } while (0)

  if (n_iter > 0) BSA_FETCH(0);
  for (int it = 0; it < n_iter; ++it) {
    if constexpr (!XT) stage_kcont<G>(rx, lds_x, lane); else stage_kstr<G, TILE>(rx, lds_x, lane);
    if constexpr (!YT) stage_kstr<G, TILE>(ry, lds_y, lane); else stage_kcont<G>(ry, lds_y, lane);
    // prefetch the next chunk while this one is multiplied; the last iteration re-reads itself (cache hit)
    // so that the loads stay unconditional and the staging registers never leave the register file
    const int nxt = (it + 1 < n_iter) ? it + 1 : it;
    BSA_FETCH(nxt);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
    for (int s = 0; s < G::STEPS; ++s) {
      u32x4 fx[G::NB], fy[G::NB];
#pragma unroll
      for (int b = 0; b < G::NB; ++b) {
        if constexpr (!XT) fx[b] = frag_kcont<G>(lds_x, b, s, lane); else fx[b] = frag_kstr<G, TILE>(lds_x, b, s, lane);
        if constexpr (!YT) fy[b] = frag_kstr<G, TILE>(lds_y, b, s, lane); else fy[b] = frag_kcont<G>(lds_y, b, s, lane);
      }
#pragma unroll
      for (int bj = 0; bj < G::NB; ++bj)
#pragma unroll
        for (int bi = 0; bi < G::NB; ++bi) acc[bj][bi] = Tr::mfma(fy[bj], fx[bi], acc[bj][bi]);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  }
#undef BSA_FETCH
#undef BSA_LOAD_WINDOW

  // epilogue: acc[bj][bi][r] = O[i = 32 bi + lane%32][j = 32 bj + 8 (r/4) + 4 (lane/32) + r%4]
  char *stage = lds_x;
  const int li = lane & 31, lh = lane >> 5;
#pragma unroll
  for (int bj = 0; bj < G::NB; ++bj)
#pragma unroll
    for (int bi = 0; bi < G::NB; ++bi)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int i = 32 * bi + li;
        const int j = 32 * bj + 8 * rq + 4 * lh;
        const int chunk = (j * ES) / 16, within = (j * ES) % 16;
        char *dst = stage + i * (G::OCPR * 16) + ((chunk ^ (i & (G::OCPR - 1) & 7)) * 16) + within;
        // 16-bit: rows i and i + OCPR share a chunk position; put their 8-byte pieces in opposite halves
        if constexpr (ES == 2) dst = stage + i * (G::OCPR * 16) + ((chunk ^ (i & (G::OCPR - 1) & 7)) * 16) +
                                     (within ^ (((i / G::OCPR) & 1) * 8));
        if constexpr (ES == 2) {
          uint2 v;
          v.x = (uint32_t)Tr::round(acc[bj][bi][4 * rq]) | ((uint32_t)Tr::round(acc[bj][bi][4 * rq + 1]) << 16);
          v.y = (uint32_t)Tr::round(acc[bj][bi][4 * rq + 2]) | ((uint32_t)Tr::round(acc[bj][bi][4 * rq + 3]) << 16);
          *reinterpret_cast<uint2 *>(dst) = v;
        } else {
          float4 v;
          v.x = acc[bj][bi][4 * rq];
          v.y = acc[bj][bi][4 * rq + 1];
          v.z = acc[bj][bi][4 * rq + 2];
          v.w = acc[bj][bi][4 * rq + 3];
          *reinterpret_cast<float4 *>(dst) = v;
        }
      }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  char *ob = out + n * block_bytes + (int64_t)ti * TILE * (int64_t)ld_bytes + (int64_t)tj * TILE * ES;
#pragma unroll
  for (int t = 0; t < G::OUT_STORES; ++t) {
    const int q = t * 64 + lane;
    const int row = q / G::OCPR, chunk = q % G::OCPR;
    u32x4 v =
        *reinterpret_cast<const u32x4 *>(stage + row * (G::OCPR * 16) + ((chunk ^ (row & (G::OCPR - 1) & 7)) * 16));
    if constexpr (ES == 2) {
      if ((row / G::OCPR) & 1) v = u32x4{v[2], v[3], v[0], v[1]};
    }
    *reinterpret_cast<u32x4 *>(ob + row * ld_bytes + chunk * 16) = v;
  }
}

// sbs == 16: one wave per output block, fp32 FMAs; lane -> row lane/4, columns 4*(lane%4)..+3
template <typename Tr>
__global__ __launch_bounds__(256) void matmul_small_kernel(const typename Tr::store_t *__restrict__ x,
                                                           const typename Tr::store_t *__restrict__ y,
                                                           typename Tr::store_t *__restrict__ out,
                                                           const int32_t *__restrict__ pair_offsets,
                                                           const int32_t *__restrict__ pairs, int64_t nnz_o,
                                                           int64_t nnz_x, int64_t nnz_y, int xt, int yt) {
  __shared__ float sx[4][16][17];
  __shared__ float sy[4][16][20];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t n = (int64_t)blockIdx.x * 4 + wave;
  if (n >= nnz_o) return;
  const int p_begin = pair_offsets[n], p_end = pair_offsets[n + 1];
  const int i = lane >> 2, j0 = (lane & 3) * 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int p = p_begin; p < p_end; ++p) {
    int64_t px = pairs[2 * (int64_t)p], py = pairs[2 * (int64_t)p + 1];
    if (px < 0 || px >= nnz_x) px = 0;
    if (py < 0 || py >= nnz_y) py = 0;
    const typename Tr::store_t *xb = x + px * 256 + lane * 4;
    const typename Tr::store_t *yb = y + py * 256 + lane * 4;
    // each lane moves 4 consecutive elements (row lane/4, columns 4*(lane%4)..) of both blocks
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float xv = Tr::widen(xb[e]);
      const float yv = Tr::widen(yb[e]);
      if (xt) sx[wave][j0 + e][i] = xv; else sx[wave][i][j0 + e] = xv;
      if (yt) sy[wave][j0 + e][i] = yv; else sy[wave][i][j0 + e] = yv;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const float a = sx[wave][i][k];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(a, sy[wave][k][j0 + e], acc[e]);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  }
  typename Tr::store_t *ob = out + n * 256 + lane * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e) ob[e] = Tr::round(acc[e]);
}

// sbs == 16, 16-bit elements: one 16 x 16 x 16 matrix-core product per pair.  A block is 512 bytes and an output
// block has one or two pairs, so a wave that handled a single block would be a chain of dependent loads
// (offsets -> pairs -> operands -> store) and nothing else.  Here a wave owns a run of consecutive output blocks,
// whose pairs are one contiguous range of the pair list: it reads that range and the run's offsets once (one
// entry per lane), then walks the pairs with the operand loads of the next two pairs in flight.
// The product is formed transposed (A = y fragment, B = x fragment), which leaves four consecutive output columns
// of one row in each lane: the wave's 8-byte stores cover the whole output block.  One 16-byte load per lane
// fetches both operand blocks of a pair (lanes 0-31 the x block, lanes 32-63 the y block: one memory instruction
// per pair instead of two, which is what the kernel's time follows); both pass through 1 KiB of LDS, from which
// an operand whose contraction index is contiguous in memory (x, or y when it is used transposed) is read as it
// lies and the other one through the transposing read.
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

struct Bf16Small {
  __device__ static f32x4 mfma(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4, a), __builtin_bit_cast(i16x4, b), c, 0, 0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    return (uint32_t)Bf16Traits::round(lo) | ((uint32_t)Bf16Traits::round(hi) << 16);
  }
};
struct F16Small {
  __device__ static f32x4 mfma(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    return (uint32_t)F16Traits::round(lo) | ((uint32_t)F16Traits::round(hi) << 16);
  }
};

constexpr int kSmallDepth = 2;    // pairs whose operand loads are in flight
constexpr int kSmallRunMax = 63;  // output blocks per wave: their offsets (one more) fit one entry per lane

// The output of a run as a buffer resource: the block's byte offset travels in a scalar register (`soffset`) and
// the lane's offset inside a block is a constant, so a store needs no per-lane address arithmetic.
__device__ inline __amdgpu_buffer_rsrc_t small_resource(const char *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base), 0, (int)bytes, 0x00020000);
}

template <typename Ts, bool XT, bool YT>
__global__ __launch_bounds__(256) void matmul_small16_kernel(const char *__restrict__ x, const char *__restrict__ y,
                                                             char *__restrict__ out,
                                                             const int32_t *__restrict__ pair_offsets,
                                                             const int32_t *__restrict__ pairs, int64_t nnz_o,
                                                             int64_t nnz_x, int64_t nnz_y, int run) {
  __shared__ __attribute__((aligned(16))) char stage[4][1024];  // per wave: the x block, then the y block
  const int lane = threadIdx.x & 63;
  // everything that steers the loops below is built from values the compiler knows to be the same in all lanes
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // workgroup g runs on XCD g % 8: every XCD takes a contiguous eighth of the runs, so that the operand blocks in
  // flight on one L2 belong to few batch entries
  const int64_t group = (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int64_t n0 = (group * 4 + wave) * run;
  if (n0 >= nnz_o) return;
  const int count = (int)(nnz_o - n0 < run ? nnz_o - n0 : run);
  // fragment of a k-contiguous operand: row lane % 16, values 4 (lane / 16) .. + 3
  const int direct_off = (lane & 15) * 32 + (lane >> 4) * 8;
  // the other operand is read transposed: inside a group of 16 lanes, lane s points at row
  // 4 (lane / 16) + s / 4, values 4 (s % 4) .. + 3
  const int turned_off = (4 * (lane >> 4) + ((lane & 15) >> 2)) * 32 + (lane & 3) * 8;
  char *slot = stage[wave];
  const uint32_t nx = (uint32_t)nnz_x, ny = (uint32_t)nnz_y;  // the pair list holds 32-bit indices
  const __amdgpu_buffer_rsrc_t ro = small_resource(out + n0 * 512, (uint32_t)count * 512u);

  // offsets of the run (count + 1 of them), one per lane
  const int off_win = pair_offsets[n0 + (lane <= count ? lane : count)];
  const int p_first = __builtin_amdgcn_readlane(off_win, 0);
  const int p_last = __builtin_amdgcn_readlane(off_win, count);

  f32x4 acc{0.f, 0.f, 0.f, 0.f};
  int done = 0;                                           // output blocks of the run already stored
  int block_end = __builtin_amdgcn_readlane(off_win, 1);  // end of the pairs of block `done`
  auto flush_until = [&](int p) {
    // store every block whose pairs end at or before p (blocks without pairs become zeros)
    while (done < count && block_end <= p) {
      u32x2 w;
      w[0] = Ts::pack2(acc[0], acc[1]);
      w[1] = Ts::pack2(acc[2], acc[3]);
      // written once, not read back by this kernel: past the caches
      __builtin_amdgcn_raw_buffer_store_b64(w, ro, direct_off, done * 512, 2);
      acc = f32x4{0.f, 0.f, 0.f, 0.f};
      ++done;
      block_end = __builtin_amdgcn_readlane(off_win, done + 1 <= count ? done + 1 : count);
    }
  };

  // the pairs of the run, 64 at a time: one entry per lane, handed out with readlane
  for (int base = p_first; base < p_last; base += 64) {
    const int n = p_last - base < 64 ? p_last - base : 64;
    u32x2 win{0u, 0u};
    if (lane < n) win = *reinterpret_cast<const u32x2 *>(pairs + 2 * (int64_t)(base + lane));
    auto issue = [&](int i, u32x4 &xy) {
      // past the end: the last pair again (a cache hit), so that every step issues the same loads and the
      // compiler can count the loads in flight instead of waiting for all of them in front of every use
      const int at = i < n ? i : n - 1;
      const uint32_t px = (uint32_t)__builtin_amdgcn_readlane((int)win[0], at);
      const uint32_t py = (uint32_t)__builtin_amdgcn_readlane((int)win[1], at);
      // a corrupt list must not turn into a wild read: such a pair reads block 0
      const char *xb = x + (int64_t)(px < nx ? px : 0) * 512;
      const char *yb = y + (int64_t)(py < ny ? py : 0) * 512;
      const char *mine = (lane < 32 ? xb : yb) + (lane & 31) * 16;
      xy = *reinterpret_cast<const u32x4 *>(mine);
    };
    u32x4 xys[kSmallDepth];
#pragma unroll
    for (int d = 0; d < kSmallDepth; ++d) issue(d, xys[d]);
    for (int i = 0; i < n; i += kSmallDepth) {
#pragma unroll
      for (int d = 0; d < kSmallDepth; ++d) {
        if (i + d < n) {
          flush_until(base + i + d);
          *reinterpret_cast<u32x4 *>(slot + lane * 16) = xys[d];
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          u32x2 fx, fy;
          if (XT) fx = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)(slot + turned_off)));
          else fx = *reinterpret_cast<const u32x2 *>(slot + direct_off);
          if (YT) fy = *reinterpret_cast<const u32x2 *>(slot + 512 + direct_off);
          else fy = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)(slot + 512 + turned_off)));
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          acc = Ts::mfma(fy, fx, acc);
        }
        issue(i + d + kSmallDepth, xys[d]);
      }
    }
  }
  flush_until(p_last);
}

template <typename Tr, int TILE>
int launch_mfma(const void *x, const void *y, void *out, const int32_t *pair_offsets, const int32_t *pairs,
                const int32_t *block_order, int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs, int trans_x,
                int trans_y, hipStream_t s) {
  const int side = sbs / TILE;
  int side_log2 = 0;
  while ((1 << side_log2) < side) ++side_log2;
  const int64_t n_tiles = nnz_o * side * side;
  // a multiple of 8 workgroups so that every XCD owns the same number of list positions
  const int64_t blocks = bsa::cdiv(bsa::cdiv(n_tiles, 4), 8) * 8;
  if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_matmul: too many output tiles");
  const char *xc = static_cast<const char *>(x);
  const char *yc = static_cast<const char *>(y);
  char *oc = static_cast<char *>(out);
#define BSA_MM_LAUNCH(XT, YT)                                                                                      \
  matmul_mfma_kernel<Tr, TILE, XT, YT><<<(unsigned)blocks, 256, 0, s>>>(xc, yc, oc, pair_offsets, pairs, block_order, \
                                                                        n_tiles, sbs, side_log2, nnz_x, nnz_y)
  if (!trans_x && !trans_y) BSA_MM_LAUNCH(false, false);
  else if (!trans_x && trans_y) BSA_MM_LAUNCH(false, true);
  else if (trans_x && !trans_y) BSA_MM_LAUNCH(true, false);
  else BSA_MM_LAUNCH(true, true);
#undef BSA_MM_LAUNCH
  return bsa::check_launch("matmul_mfma_kernel");
}

template <typename Tr>
int launch_any(const void *x, const void *y, void *out, const int32_t *pair_offsets, const int32_t *pairs,
               const int32_t *block_order, int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs, int trans_x,
               int trans_y, hipStream_t s) {
  if (sbs == 16 && Tr::kElem == 2) {
    using Ts = std::conditional_t<std::is_same_v<Tr, Bf16Traits>, Bf16Small, F16Small>;
    // enough waves to fill the chip, each with a run long enough to overlap its loads
    int64_t run = bsa::cdiv(nnz_o, 256 * 32 * 4);
    run = run < 8 ? 8 : (run > kSmallRunMax ? kSmallRunMax : run);
    const int64_t blocks = bsa::cdiv(bsa::cdiv(bsa::cdiv(nnz_o, run), 4), 8) * 8;
    if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_matmul: too many output blocks");
    const char *xc = static_cast<const char *>(x);
    const char *yc = static_cast<const char *>(y);
    char *oc = static_cast<char *>(out);
#define BSA_MM_SMALL(XT, YT)                                                                                        \
  matmul_small16_kernel<Ts, XT, YT><<<(unsigned)blocks, 256, 0, s>>>(xc, yc, oc, pair_offsets, pairs, nnz_o, nnz_x, \
                                                                     nnz_y, (int)run)
    if (!trans_x && !trans_y) BSA_MM_SMALL(false, false);
    else if (!trans_x && trans_y) BSA_MM_SMALL(false, true);
    else if (trans_x && !trans_y) BSA_MM_SMALL(true, false);
    else BSA_MM_SMALL(true, true);
#undef BSA_MM_SMALL
    return bsa::check_launch("matmul_small16_kernel");
  }
  if (sbs == 16) {
    using E = typename Tr::store_t;
    const int64_t blocks = bsa::cdiv(nnz_o, 4);
    if (blocks > 0x7fffffffLL) return bsa::fail(BSA_ELIMIT, "bsa_matmul: too many output blocks");
    matmul_small_kernel<Tr><<<(unsigned)blocks, 256, 0, s>>>(static_cast<const E *>(x), static_cast<const E *>(y),
                                                             static_cast<E *>(out), pair_offsets, pairs, nnz_o,
                                                             nnz_x, nnz_y, trans_x, trans_y);
    return bsa::check_launch("matmul_small_kernel");
  }
  if (sbs == 32)
    return launch_mfma<Tr, 32>(x, y, out, pair_offsets, pairs, block_order, nnz_o, nnz_x, nnz_y, sbs, trans_x, trans_y, s);
  return launch_mfma<Tr, 64>(x, y, out, pair_offsets, pairs, block_order, nnz_o, nnz_x, nnz_y, sbs, trans_x, trans_y, s);
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int bsa_matmul(const void *x, const void *y, void *out, const int32_t *pair_offsets, const int32_t *pairs,
                          const int32_t *block_order, int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs, int dtype, int trans_x, int trans_y,
                          bsa_stream_t stream) {
  BSA_REQUIRE(sbs >= 16 && bsa::is_pow2(sbs), "bsa_matmul: sbs must be a power of two >= 16 (got %d)", sbs);
  BSA_REQUIRE(nnz_o >= 0 && nnz_x >= 0 && nnz_y >= 0, "bsa_matmul: negative size");
  BSA_REQUIRE(dtype == BSA_F32 || dtype == BSA_F16 || dtype == BSA_BF16, "bsa_matmul: unknown dtype %d", dtype);
  if (nnz_o == 0) return BSA_OK;
  BSA_REQUIRE(out && pair_offsets, "bsa_matmul: NULL pointer");
  BSA_REQUIRE(aligned16(x) && aligned16(y) && aligned16(out), "bsa_matmul: buffers must be 16-byte aligned");
  hipStream_t s = bsa::as_stream(stream);
  switch (dtype) {
    case BSA_BF16:
      return launch_any<Bf16Traits>(x, y, out, pair_offsets, pairs, block_order, nnz_o, nnz_x, nnz_y, sbs, trans_x, trans_y, s);
    case BSA_F16:
      return launch_any<F16Traits>(x, y, out, pair_offsets, pairs, block_order, nnz_o, nnz_x, nnz_y, sbs, trans_x, trans_y, s);
    default:
      return launch_any<F32Traits>(x, y, out, pair_offsets, pairs, block_order, nnz_o, nnz_x, nnz_y, sbs, trans_x, trans_y, s);
  }
}
