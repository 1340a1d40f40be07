// Block-sparse flash attention backward on the matrix cores: fp16 / bf16 operands, sbs == 64, one or two
// 64-wide head slices for q/k and for v/o.
//
// Three kernels, as in the reference (blksprs/ops/flash_attention.py:1235-1735): delta = rowsum(o * dO);
// dK / dV (and dBias) per key block, walking the query blocks that attend to it; dQ per query block, walking
// its key blocks.  The two main kernels recompute the scores and probabilities of a (query block, key block)
// pair from the saved log-sum-exp, in the same order as the forward kernel: scale * q k^T, + bias, native causal
// predicate, explicit mask.  Probabilities and dS are rounded to the operand type before they enter a product.
//
// Both main kernels have the same shape.  One workgroup of four waves owns the "stationary" block (a key block,
// or a query block); each wave owns one 32 x 32 quadrant of the 64 x 64 score tile and keeps the fragments of
// its half of the stationary operands in registers for the whole walk.  The blocks of the other side stream
// through LDS, double buffered, one barrier per tile, copied global -> LDS asynchronously, row-major with
// XOR-swizzled 16-byte chunks.  A matrix-core operand wants eight consecutive contraction indices per lane:
// where the head dimension is contracted (scores, dP) a fragment is one 128-bit read of a row, where the
// sequence index is contracted (dV, dK, dQ) it is two transposing 64-bit reads (ds_read_b64_tr_b16).
//
//   dK / dV kernel, lane owns a key j, registers run over queries i:
//     S[i][j]  = sum_d Q[i][d] K[j][d]        A = Q rows (LDS)     B = K (registers)
//     dP[i][j] = sum_d dO[i][d] V[j][d]       A = dO rows (LDS)    B = V (registers)
//     dV^T[d][j] += sum_i dO[i][d] P[i][j]    A = dO columns (LDS) B = P (registers, as computed)
//     dK^T[d][j] += sum_i Q[i][d] dS[i][j]    A = Q columns (LDS)  B = dS
//   dQ kernel, lane owns a query i, registers run over keys j:
//     S^T[j][i], dP^T[j][i] likewise with K, V rows from LDS and Q, dO in registers
//     dQ^T[d][i] += sum_j K[j][d] dS^T[j][i]  A = K columns (LDS)  B = dS^T
//
// The two waves that share a half of the stationary block hold partial sums over the two halves of the streamed
// blocks; they are added through LDS once, at the end.  No atomics, fixed summation order.
#include <atomic>
#include <type_traits>

#include "attn_mfma_common.h"

namespace bsa {
namespace {

using namespace mfma;

constexpr int kBwdThreads = 256;
constexpr int kStatBytes = 2 * kSbs * 4;  // lse and delta of the 64 queries of a tile
// One 64 x 64 16-bit block, global -> LDS, by the NW (4 or 8) waves of a workgroup: wave w copies rows
// (64 / NW) w .. with asynchronous 1 KiB copies (eight rows each); lane l supplies the chunk that belongs at
// position l of the KiB, which is where the chunk swizzle is applied.  An inactive block becomes zeros.
template <int NW = 4>
__device__ inline void copy_block(const char *blk, bool valid, char *dst, int wave, int lane, int tid) {
  constexpr int kCopies = 8 / NW;  // KiB per wave
  if (valid) {
#pragma unroll
    for (int i = 0; i < kCopies; ++i) {
      const int r0 = 8 * kCopies * wave + 8 * i;
      const uint32_t lane_off = (lane >> 3) * 128 + (((lane & 7) ^ t_swizzle(8 * i + (lane >> 3))) << 4);
      copy_1k_to_lds(blk + r0 * 128, lane_off, dst + r0 * 128);
    }
  } else {
#pragma unroll
    for (int i = 0; i < kCopies; ++i) *reinterpret_cast<u32x4 *>(dst + (i * NW * 64 + tid) * 16) = u32x4{0u, 0u, 0u, 0u};
  }
}

// operand fragment with the head dimension contracted: 8 values of row `row`, 16-byte chunk `chunk`
__device__ inline u32x4 frag_rows(const char *lds, int row, int chunk) {
  return *reinterpret_cast<const u32x4 *>(lds + row * 128 + ((chunk ^ t_swizzle(row)) << 4));
}

// fragment of a block in global memory for the register-resident side: row `row`, chunks 2 s + kg
__device__ inline void load_resident(u32x4 (&f)[4], const void *base, int64_t pidx, int64_t n_blocks, int row, int kg) {
  const bool valid = pidx >= 0 && pidx < n_blocks;
  const char *p = static_cast<const char *>(base) + (valid ? pidx : 0) * kBlockBytes + row * 128 + kg * 16;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    f[s] = u32x4{0u, 0u, 0u, 0u};
    if (valid) f[s] = *reinterpret_cast<const u32x4 *>(p + 32 * s);
  }
}

// A run of matrix-core products whose A operands come from LDS, four fragments to a stage: the reads of stage
// k + 1 are issued before the products of stage k, so that a read's latency is paid behind four products and not
// in front of each one.  `load(k, f)` fills the four fragments of stage k, `multiply(k, f)` consumes them.  The
// empty statement that names a fragment keeps its read from sinking to its use.
template <int K, typename Load, typename Multiply>
__device__ __forceinline__ void staged_products(Load load, Multiply multiply) {
  u32x4 f[2][4];
  load(0, f[0]);
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (k + 1 < K) load(k + 1, f[(k + 1) & 1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(f[k & 1][i]));
    multiply(k, f[k & 1]);
  }
}

// workgroups per XCD of the dK / dV kernel whose workgroups stay for the whole launch: one per compute unit
constexpr int kCusPerXcd = 32;
__host__ __device__ inline int64_t kv_slots(int64_t key_rows) {
  const int64_t chunk = (key_rows + 7) / 8;
  return chunk < kCusPerXcd ? chunk : kCusPerXcd;
}

// The same run with the fragments of stage 0 already requested by the caller (`first`), so that their latency
// lies behind whatever the caller did in between.
template <int K, typename Load, typename Multiply>
__device__ __forceinline__ void staged_products_from(const u32x4 (&first)[4], Load load, Multiply multiply) {
  u32x4 f[2][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) f[0][i] = first[i];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (k + 1 < K) load(k + 1, f[(k + 1) & 1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(f[k & 1][i]));
    multiply(k, f[k & 1]);
  }
}

// XCD-aware row of a workgroup: every XCD gets a contiguous range of rows, so that the blocks in flight on one
// L2 belong to the same batch entries
__device__ inline int64_t xcd_row() { return (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3); }

// sum of the accumulators of wave pairs (w, w ^ partner_bit): the wave with the bit set writes, the other adds
template <int N>
__device__ inline void reduce_partner(f32x16 (&acc)[N], float *lds, bool writer, int slot, int lane) {
  // slot: which pair of waves (0 or 1); layout [slot][n][r / 4][lane][r % 4]: 128-bit accesses, a wave's lanes side
  // by side
  f32x4 *base = reinterpret_cast<f32x4 *>(lds + (size_t)slot * N * 16 * 64) + lane;
  __syncthreads();  // the tile buffers are free
  if (writer) {
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        base[(n * 4 + q) * 64] = f32x4{acc[n][4 * q], acc[n][4 * q + 1], acc[n][4 * q + 2], acc[n][4 * q + 3]};
  }
  __syncthreads();
  if (!writer) {
#pragma unroll
    for (int n = 0; n < N; ++n)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4 v = base[(n * 4 + q) * 64];
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[n][4 * q + t] += v[t];
      }
  }
}

// The same sum, shared out between the two waves of a pair: of the accumulators 2 h and 2 h + 1 (the two column
// halves of slice h) each wave gives one away and adds what it gets to the other, so both move and add half as
// much and both end with a finished half.  The caller has put the half it keeps into the EVEN accumulators (the
// wave with partner bit 1 swaps its pairs first), so that one copy of these loops serves both waves.
// Layout [slot][giver][h][r / 4][lane][r % 4].
template <int N>
__device__ inline void exchange_odd_for_even(f32x16 (&acc)[N], float *lds, int giver, int slot, int lane) {
  static_assert(N % 2 == 0, "pairs of accumulators");
  constexpr int kPerWave = (N / 2) * 16 * 64;
  f32x4 *give = reinterpret_cast<f32x4 *>(lds + (size_t)(slot * 2 + giver) * kPerWave) + lane;
  const f32x4 *take = reinterpret_cast<const f32x4 *>(lds + (size_t)(slot * 2 + (1 - giver)) * kPerWave) + lane;
  __syncthreads();  // the tile buffers are free
#pragma unroll
  for (int h = 0; h < N / 2; ++h)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x16 &out = acc[2 * h + 1];
      give[(h * 4 + q) * 64] = f32x4{out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
    }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < N / 2; ++h)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x4 v = take[(h * 4 + q) * 64];
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[2 * h][4 * q + t] += v[t];
    }
}

// ---------------------------------------------------------------------------------------------------------
// Records of the pairs that can contribute.  A (query block, key block) pair whose mask block masks every score,
// or that the causal predicate rules out as a whole, has P = dS = 0.  Which pairs those are depends on the mask's
// contents, so it is found out at the start of every backward call: one pass over the mask blocks, then the
// two lists of the attention layout (key blocks per query block, query blocks per key block) are written out
// without the dead pairs, in the same order, each entry as a record that already holds every index its tile
// needs.  The two main kernels walk those records: one 32-byte load per tile instead of a chain of gathers.
struct BwdRecord {
  int32_t other;   // the query block (lists per key block) or key block (lists per query block)
  int32_t pa[2];   // packed indices of its Q (resp. K) slices, -1: none
  int32_t pb[2];   // packed indices of its O / dO (resp. V) slices
  int32_t mask;    // mask block of the pair, -1: none
  int32_t bias;    // bias block of the pair
  int32_t pair;    // position of the pair in key_indices (the same number in both lists): its block of dS
};
static_assert(sizeof(BwdRecord) == 32, "one record is eight int32");

struct BwdLists {
  BwdRecord *key_rec, *query_rec;  // [n_layout_blocks] each, rows at the offsets of key_offsets / query_offsets
  int32_t *key_end, *query_end;    // [B * nq], [B * nk]: end of the live part of a row's list
  // [B * nq][16], [B * nk][16]: one 64-byte header per workgroup of the dQ resp. dK / dV kernel, in the order in
  // which rows are handed out: ints 0 .. 7 the first record of the row's list, 8 the row, 9 and 10 the bounds of
  // its live list, 11 .. 12 and 13 .. 14 the packed indices of the stationary block's slices (Q and O for a
  // query row, K and V for a key row; -1: none).  Everything a workgroup has to know before its first tile
  // comes with one load.
  int32_t *q_head, *k_head;
  int32_t *kv_tickets;             // [16]: per XCD, the next position of its eighth of the key rows to hand out
  uint8_t *mask_dead;              // [n_mask_blocks]
  // [n_layout_blocks] blocks of 64 x 64 16-bit values, or NULL (the caller brought no room for them): dS^T of every
  // pair (row = key, column = query), written by the dK / dV kernel for the dQ kernel
  char *ds;
};

// bytes of the scratch (the dS blocks have a buffer of their own, bsa_attn_args.bwd_ds)
__host__ __device__ inline size_t bwd_lists_bytes(int64_t B, int64_t nq, int64_t nk, int64_t n_layout_blocks,
                                                  int64_t n_mask_blocks) {
  const size_t bytes = 2 * sizeof(BwdRecord) * (size_t)n_layout_blocks + (4 + 64) * (size_t)(B * nq + B * nk) + 64 +
                       (size_t)n_mask_blocks;
  return (bytes + 15) & ~(size_t)15;
}
__host__ __device__ inline BwdLists bwd_lists(const bsa_attn_args &a) {
  BwdLists L;
  L.key_rec = static_cast<BwdRecord *>(a.bwd_scratch);
  L.query_rec = L.key_rec + a.n_layout_blocks;
  L.key_end = reinterpret_cast<int32_t *>(L.query_rec + a.n_layout_blocks);
  L.query_end = L.key_end + a.B * a.nq;
  L.q_head = L.query_end + a.B * a.nk;
  L.k_head = L.q_head + 16 * a.B * a.nq;
  L.kv_tickets = L.k_head + 16 * a.B * a.nk;
  L.mask_dead = reinterpret_cast<uint8_t *>(L.kv_tickets + 16);
  const bool has_ds = a.bwd_ds != nullptr && a.bwd_ds_bytes >= a.n_layout_blocks * (int64_t)kBlockBytes;
  L.ds = has_ds ? static_cast<char *>(a.bwd_ds) : nullptr;
  return L;
}

// one wave per mask block (4 KiB of bytes 0 / 1)
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_mask_dead_kernel(const u32x4 *mask, uint8_t *dead, int64_t n) {
  const int64_t m = ((int64_t)blockIdx.x * kBwdThreads + threadIdx.x) >> 6;
  if (m >= n) return;
  const int lane = threadIdx.x & 63;
  const u32x4 *p = mask + m * (kSbs * kSbs / 16);
  uint32_t all = 0x01010101u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const u32x4 v = p[i * 64 + lane];
    all &= v[0] & v[1] & v[2] & v[3];
  }
  const unsigned long long votes = __ballot(all == 0x01010101u);
  if (lane == 0) dead[m] = votes == ~0ull ? 1 : 0;
}

__device__ inline int32_t checked_index(const int64_t *table, int64_t at, int64_t n) {
  const int64_t v = table[at];
  return (v >= 0 && v < n) ? (int32_t)v : -1;
}

// One wave per query block row (by_key false), in a second launch one per key block row (by_key true): the lists
// per key block name every pair by its position in the finished list of its query block.
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_records_kernel(bsa_attn_args a, bool by_key) {
  const int64_t w = ((int64_t)blockIdx.x * kBwdThreads + threadIdx.x) >> 6;
  if (w >= (by_key ? a.B * a.nk : a.B * a.nq)) return;
  const int lane = threadIdx.x & 63;
  const BwdLists L = bwd_lists(a);
  const int64_t row = w;
  const int64_t per_batch = by_key ? a.nk : a.nq;
  const int64_t b = row / per_batch, mine = row % per_batch;
  const int32_t *offsets = by_key ? a.query_offsets : a.key_offsets;
  const int32_t *indices = by_key ? a.query_indices : a.key_indices;
  BwdRecord *out = by_key ? L.query_rec : L.key_rec;
  const bool causal = a.causal_lengths != nullptr;
  const int64_t seq_len = causal ? a.causal_lengths[b] : 0;
  const int begin = offsets[row], end = offsets[row + 1];
  // does some score of the pair survive?  pm: its mask block
  auto pair_live = [&](int64_t qb, int64_t kb, int32_t &pm) -> bool {
    pm = -1;
    if (causal && (kb > qb || qb * kSbs >= seq_len || kb * kSbs >= seq_len)) return false;
    if (a.mask) {
      pm = checked_index(a.pidx_mask, (b * a.nq + qb) * a.nk + kb, a.n_mask_blocks);
      if (pm >= 0 && L.mask_dead[pm]) return false;
    }
    return true;
  };
  int n = begin;
  for (int e0 = begin; e0 < end; e0 += 64) {
    const int e = e0 + lane;
    bool live = e < end;
    const int64_t other = live ? indices[e] : 0;
    const int64_t qb = by_key ? other : mine, kb = by_key ? mine : other;
    const int64_t pair = (b * a.nq + qb) * a.nk + kb;
    int32_t pm = -1;
    if (live) live = pair_live(qb, kb, pm);
    const unsigned long long votes = __ballot(live);
    if (live) {
      BwdRecord r;
      r.other = (int32_t)other;
      // what streams past the stationary block: Q and dO of the query block, or K and V of the key block
      const int64_t orow = by_key ? b * a.nq + qb : b * a.nk + kb;
      const int64_t *ta = by_key ? a.pidx_q : a.pidx_k, *tb = by_key ? a.pidx_o : a.pidx_v;
      const int64_t na = by_key ? a.n_q_blocks : a.n_k_blocks, nb = by_key ? a.n_o_blocks : a.n_v_blocks;
      for (int h = 0; h < 2; ++h) {
        r.pa[h] = h < a.nh ? checked_index(ta, orow * a.nh + h, na) : -1;
        r.pb[h] = h < a.nhv ? checked_index(tb, orow * a.nhv + h, nb) : -1;
      }
      r.mask = pm;
      r.bias = a.bias ? checked_index(a.pidx_bias, pair, a.n_bias_blocks) : -1;
      // the pair's position in the list of its query block as written by the first launch (without the dead
      // pairs): where this record goes, or, from the side of the key block, where the query block's list, which is
      // sorted by key block, holds this key block (a pair is live from both sides or from neither)
      int at = n + __popcll(votes & ((1ull << lane) - 1));
      if (by_key) {
        const int64_t qrow = b * a.nq + qb;
        int lo = a.key_offsets[qrow], hi = L.key_end[qrow];
        while (lo < hi) {
          const int mid = lo + ((hi - lo) >> 1);
          if (L.key_rec[mid].other < (int32_t)kb) lo = mid + 1;
          else hi = mid;
        }
        // lists that do not match each other must not turn into a position outside the dS blocks
        at = lo < a.n_layout_blocks ? lo : (int)a.n_layout_blocks - 1;
      }
      r.pair = at;
      out[n + __popcll(votes & ((1ull << lane) - 1))] = r;
    }
    n += __popcll(votes);
  }
  if (lane == 0) (by_key ? L.query_end : L.key_end)[row] = n;
}

// Workgroup g of a main kernel runs on XCD g % 8, and every XCD is given a contiguous eighth of the rows, so that
// the blocks in flight on one L2 belong to the same batch entries.  Inside its eighth an XCD takes first the few
// rows with more than four times the mean number of live pairs (a row that every query attends to can be a hundred
// times longer than the others and must not be the last to start), then all the others, both groups in their
// natural order: neighbouring rows share most of the blocks they stream (a local window of +-w blocks has 2 w of
// its 2 w + 1 tiles in common with the next row's), and rows handed out one after the other are in flight together,
// so those tiles are fetched from memory once and found in the L2 afterwards.  (Ordering all rows by length
// scatters the neighbours over the launch: on a window + global + random layout the dK / dV walk then fetched twice
// the bytes.)  The order is a stable partition, the same on every run.  Workgroups 0 .. 7 order the query rows,
// 8 .. 15 the key rows.  What is written per position is the 64-byte header of the workgroup that takes it.
constexpr int kOrderThreads = 1024;
__global__ __launch_bounds__(kOrderThreads) void attn_bwd_order_kernel(bsa_attn_args a) {
  const BwdLists L = bwd_lists(a);
  const bool by_key = blockIdx.x >= 8;
  const int64_t rows = by_key ? a.B * a.nk : a.B * a.nq;
  const int32_t *offsets = by_key ? a.query_offsets : a.key_offsets;
  const int32_t *ends = by_key ? L.query_end : L.key_end;
  int32_t *heads = by_key ? L.k_head : L.q_head;
  const BwdRecord *recs = by_key ? L.query_rec : L.key_rec;
  const int64_t *ta = by_key ? a.pidx_k : a.pidx_q, *tb = by_key ? a.pidx_v : a.pidx_o;
  const int64_t na = by_key ? a.n_k_blocks : a.n_q_blocks, nb = by_key ? a.n_v_blocks : a.n_o_blocks;
  auto emit = [&](int64_t pos, int64_t r) {
    int32_t *h = heads + pos * 16;
    const int begin = offsets[r], end = ends[r];
    const int32_t *first = reinterpret_cast<const int32_t *>(recs + begin);
    for (int i = 0; i < 8; ++i) h[i] = begin < end ? first[i] : -1;
    h[8] = (int32_t)r;
    h[9] = begin;
    h[10] = end;
    for (int s = 0; s < 2; ++s) {
      h[11 + s] = s < a.nh ? checked_index(ta, r * a.nh + s, na) : -1;
      h[13 + s] = s < a.nhv ? checked_index(tb, r * a.nhv + s, nb) : -1;
    }
    h[15] = 0;
  };
  const int64_t chunk = (rows + 7) / 8;  // = gridDim.x / 8 of the main kernels
  const int64_t r0 = (int64_t)(blockIdx.x & 7) * chunk, r1 = r0 + chunk < rows ? r0 + chunk : rows;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  __shared__ unsigned long long total;
  __shared__ int n_long;
  __shared__ int wave_long[kOrderThreads / 64];
  if (tid == 0) {
    total = 0;
    n_long = 0;
  }
  __syncthreads();
  unsigned long long mine = 0;
  for (int64_t r = r0 + tid; r < r1; r += kOrderThreads) mine += (unsigned long long)(ends[r] - offsets[r]);
  if (mine) atomicAdd(&total, mine);
  __syncthreads();
  const unsigned long long sum = total, count = r0 < r1 ? (unsigned long long)(r1 - r0) : 0ull;
  auto is_long = [&](int64_t r) { return (unsigned long long)(ends[r] - offsets[r]) * count > 4ull * sum; };
  int mine_long = 0;
  for (int64_t r = r0 + tid; r < r1; r += kOrderThreads) mine_long += is_long(r) ? 1 : 0;
  if (mine_long) atomicAdd(&n_long, mine_long);
  __syncthreads();
  const int64_t longs = n_long;
  if (longs == 0) {
    for (int64_t r = r0 + tid; r < r1; r += kOrderThreads) emit(r, r);
    return;
  }
  // stable partition, 1024 rows at a time: the long rows of the tile go behind the long rows before it, the others
  // behind all long rows and the other rows before them
  int64_t long_done = 0;
  for (int64_t base = r0; base < r1; base += kOrderThreads) {
    const int64_t r = base + tid;
    const bool valid = r < r1;
    const bool lng = valid && is_long(r);
    const unsigned long long votes = __ballot(lng);
    if (lane == 0) wave_long[wave] = __popcll(votes);
    __syncthreads();
    int before = __popcll(votes & ((1ull << lane) - 1)), in_tile = 0;
    for (int w = 0; w < kOrderThreads / 64; ++w) {
      before += w < wave ? wave_long[w] : 0;
      in_tile += wave_long[w];
    }
    if (valid) emit(lng ? r0 + long_done + before : r0 + longs + (base - r0 - long_done) + (tid - before), r);
    long_done += in_tile;
    __syncthreads();  // wave_long is written again
  }
}

// delta[b, qb, i] = sum over the output slices of rowsum(o * dO), four lanes per query row; also the tickets of
// the dK / dV walk.  Launched in front of that walk when the dQ kernel runs after it (dQ from the stored dS).
template <typename Tr>
__global__ __launch_bounds__(kBwdThreads) void attn_bwd_delta_kernel(bsa_attn_args a) {
  const int64_t row = blockIdx.x;  // b * nq + qb
  const int tid = threadIdx.x;
  if (row == 0 && tid < 8) bwd_lists(a).kv_tickets[tid] = (int32_t)kv_slots(a.B * a.nk);
  const int i = tid >> 2, part = tid & 3;
  float acc = 0.f;
  for (int64_t h = 0; h < a.nhv; ++h) {
    const int64_t po = a.pidx_o[row * a.nhv + h];
    if (po < 0 || po >= a.n_o_blocks) continue;
    const char *ob = static_cast<const char *>(a.o) + po * kBlockBytes + i * 128 + part * 32;
    const char *gb = static_cast<const char *>(a.d_o) + po * kBlockBytes + i * 128 + part * 32;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      // o is read here and nowhere else in the backward; dO is read again by the walk that follows: o goes past the caches
      const u32x4 ov = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(ob + 16 * c));
      const u32x4 gv = *reinterpret_cast<const u32x4 *>(gb + 16 * c);
#pragma unroll
      for (int t = 0; t < 4; ++t) acc = Tr::dot2(ov[t], gv[t], acc);
    }
  }
  acc += __shfl_xor(acc, 1);
  acc += __shfl_xor(acc, 2);
  if (part == 0) a.delta[row * kSbs + i] = acc;
}

// A tile with the work split between the two teams of the eight-wave kernel: the dV team (DV) computes S and P,
// leaves P (fp32, as computed) in LDS for the wave of the dK team that owns the same quadrant, and adds
// dV^T += dO^T P; the dK team (DK) computes dP meanwhile, reads P, forms dS = P (dP - delta) and adds
// dK^T += Q^T dS.  Each team then issues 16 products per tile (24 and 16 when both compute S) and only one of them
// the exponentials; the results are the same bits.  One barrier in the middle of the tile, passed by every wave
// whether its quadrant is live or not, hands P over; p_lds: this quadrant's 4 KiB, lane's slot ([q][lane] of 16
// bytes).  The next P is written after the barrier that ends the tile, when this one has been read.
// The tile comes in three calls, so that the caller can put other work behind the LDS reads that open each half:
// kv_first_frags requests the fragments the first products start with (the caller then requests the next tile),
// kv_first_half ends by requesting those of the second half (the caller then passes the barrier).

// A quadrant whose every score is masked has P = dS = 0: nothing to add, nothing to compute.
__device__ __forceinline__ bool kv_quadrant_live(const int64_t pm, const uint32_t mbits, const bool causal, const int kb,
                                                 const int qb, const int seq_len, const int wi, const int wj) {
  bool live = true;
  if (pm >= 0) live = !__all(mbits == 0xffffu);
  if (causal) {
    const int k_first = kb * kSbs + 32 * wj, q_first = qb * kSbs + 32 * wi;
    if (k_first > q_first + 31 || q_first >= seq_len || k_first >= seq_len) live = false;
  }
  return live;
}

// stage 0 of the first products: rows of Q (dV team: S) or of dO (dK team: dP)
template <int NH, bool DK>
__device__ __forceinline__ void kv_first_frags(u32x4 (&f0)[4], const char *base, const int wi, const int li, const int kg) {
  const char *src = base + (DK ? NH * kBlockBytes : 0);
#pragma unroll
  for (int s = 0; s < 4; ++s) f0[s] = frag_rows(src, 32 * wi + li, 2 * s + kg);
}

// what a wave carries over the barrier in the middle of the tile
struct KvCarry {
  u32x4 g0[4];   // stage 0 of the second products: columns of dO (dV team) or of Q (dK team)
  u32x4 pf[2];   // dV team: P as operand
  f32x16 dpacc;  // dK team: dP
};

template <typename Tr, int NH, int NHV, bool DK, bool DV>
__device__ __forceinline__ void kv_first_half(KvCarry &c, const u32x4 (&f0)[4], const bool live, const bsa_attn_args &a,
                                              const char *base, const int qb, const int64_t pm, const int64_t pb,
                                              const uint32_t mbits, const bool causal, const int seq_len, const int kb,
                                              const int kpos, const float qk_scale, const int wi, const int wj,
                                              const int li, const int kg, const int lane, const u32x4 (&kfr)[NH][4],
                                              const u32x4 (&vfr)[NHV][4], f32x4 *p_lds) {
  static_assert(DK != DV, "one team each");
  constexpr int kQRows = 0, kDoRows = NH * kBlockBytes, kStats = (NH + NHV) * kBlockBytes;
  if (!live) return;
  const float *stats = reinterpret_cast<const float *>(base + kStats);
  const int col_t = 16 * ((lane >> 4) & 1);
  if constexpr (DV) {
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    staged_products_from<NH>(
        f0,
        [&](int k, u32x4(&f)[4]) {
#pragma unroll
          for (int s = 0; s < 4; ++s) f[s] = frag_rows(base + kQRows + k * kBlockBytes, 32 * wi + li, 2 * s + kg);
        },
        [&](int k, u32x4(&f)[4]) {
#pragma unroll
          for (int s = 0; s < 4; ++s) sacc = Tr::mfma(f[s], kfr[k][s], sacc);
        });
    // the fragments the dV products start with: in flight while P is formed
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c.g0[i] = frag_cols_t(base + kDoRows, 32 * wi + 16 * (i & 1) + 4 * kg, 32 * (i >> 1) + col_t, lane);
    // ---- P; element r: query 32 wi + 8 (r / 4) + 4 kg + r % 4 ----
    uint32_t bias_c[16];
    if (pb >= 0) {
      const uint16_t *bp = static_cast<const uint16_t *>(a.bias) + pb * (kSbs * kSbs) +
                           (32 * wi + 4 * kg) * kSbs + 32 * wj + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) bias_c[r] = bp[(8 * (r >> 2) + (r & 3)) * kSbs];
    }
    float p[16];
    auto probabilities = [&](auto plain_tag) {
      constexpr bool kPlain = decltype(plain_tag)::value;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i0 = 32 * wi + 8 * q + 4 * kg;
        const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(stats + i0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int r = 4 * q + t;
          float s = sacc[r] * qk_scale;
          if constexpr (!kPlain) {
            if (pb >= 0) s = s + Tr::widen((uint16_t)bias_c[r]) * kLog2e;
            if (causal) {
              const int qpos = qb * kSbs + i0 + t;
              s = (kpos > qpos || qpos >= seq_len || kpos >= seq_len) ? -INFINITY : s;
            }
            if (pm >= 0) s = ((mbits >> r) & 1u) ? -INFINITY : s;
          }
          p[r] = __builtin_amdgcn_exp2f(s - lse4[t]);
        }
      }
    };
    // Most tiles have no bias, no mask block and lie where the causal predicate holds for every score: they take
    // the plain path.  The conditions are the same for the whole wave.
    bool plain = pb < 0 && pm < 0;
    if (causal) {
      const int k_last = kb * kSbs + 32 * wj + 31, q_first = qb * kSbs + 32 * wi;
      plain = plain && k_last <= q_first && q_first + 31 < seq_len;
    }
    if (plain) probabilities(std::true_type{});
    else probabilities(std::false_type{});
#pragma unroll
    for (int q = 0; q < 4; ++q) p_lds[q * 64] = f32x4{p[4 * q], p[4 * q + 1], p[4 * q + 2], p[4 * q + 3]};
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) c.pf[u][t] = Tr::pack2(p[8 * u + 2 * t], p[8 * u + 2 * t + 1]);
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) c.dpacc[r] = 0.f;
    staged_products_from<NHV>(
        f0,
        [&](int k, u32x4(&f)[4]) {
#pragma unroll
          for (int s = 0; s < 4; ++s) f[s] = frag_rows(base + kDoRows + k * kBlockBytes, 32 * wi + li, 2 * s + kg);
        },
        [&](int k, u32x4(&f)[4]) {
#pragma unroll
          for (int s = 0; s < 4; ++s) c.dpacc = Tr::mfma(f[s], vfr[k][s], c.dpacc);
        });
    // the fragments the dK products start with: in flight across the barrier and while dS is formed
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c.g0[i] = frag_cols_t(base + kQRows, 32 * wi + 16 * (i & 1) + 4 * kg, 32 * (i >> 1) + col_t, lane);
  }
}

template <typename Tr, int NH, int NHV, bool DK, bool DV>
__device__ __forceinline__ void kv_second_half(const KvCarry &c, const bool live, const bsa_attn_args &a, const char *base,
                                               const int64_t pb, const int wi, const int wj, const int li, const int kg,
                                               const int lane, f32x16 (&dkacc)[DK ? NH * 2 : 1],
                                               f32x16 (&dvacc)[DV ? NHV * 2 : 1], const f32x4 *p_lds,
                                               u32x4 (&ds_keep)[2]) {
  constexpr int kQRows = 0, kDoRows = NH * kBlockBytes, kStats = (NH + NHV) * kBlockBytes;
  // ds_keep (dK team): dS of this lane's 16 scores as packed for the dK product, zeros for a quadrant without a
  // surviving score; the caller stores it for the dQ kernel
  if constexpr (DK) ds_keep[0] = ds_keep[1] = u32x4{0u, 0u, 0u, 0u};
  if (!live) return;
  const int col_t = 16 * ((lane >> 4) & 1);
  if constexpr (DV) {
    staged_products_from<NHV>(
        c.g0,
        [&](int h, u32x4(&f)[4]) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            f[i] = frag_cols_t(base + kDoRows + h * kBlockBytes, 32 * wi + 16 * (i & 1) + 4 * kg, 32 * (i >> 1) + col_t, lane);
        },
        [&](int h, u32x4(&f)[4]) {
#pragma unroll
          for (int i = 0; i < 4; ++i) dvacc[2 * h + (i >> 1)] = Tr::mfma(f[i], c.pf[i & 1], dvacc[2 * h + (i >> 1)]);
        });
  } else {
    const float *stats = reinterpret_cast<const float *>(base + kStats);
    float ds[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i0 = 32 * wi + 8 * q + 4 * kg;
      const f32x4 del4 = *reinterpret_cast<const f32x4 *>(stats + kSbs + i0);
      const f32x4 p4 = p_lds[q * 64];
#pragma unroll
      for (int t = 0; t < 4; ++t) ds[4 * q + t] = p4[t] * (c.dpacc[4 * q + t] - del4[t]);
    }
    if (a.dbias != nullptr && pb >= 0) {
      // every (query block, key block) pair is visited once, so this is a plain store
      float *dbp = a.dbias + pb * (kSbs * kSbs) + (32 * wi + 4 * kg) * kSbs + 32 * wj + li;
#pragma unroll
      for (int r = 0; r < 16; ++r) dbp[(8 * (r >> 2) + (r & 3)) * kSbs] = ds[r];
    }
    u32x4 dsf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) dsf[u][t] = Tr::pack2(ds[8 * u + 2 * t], ds[8 * u + 2 * t + 1]);
    ds_keep[0] = dsf[0];
    ds_keep[1] = dsf[1];
    staged_products_from<NH>(
        c.g0,
        [&](int h, u32x4(&f)[4]) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            f[i] = frag_cols_t(base + kQRows + h * kBlockBytes, 32 * wi + 16 * (i & 1) + 4 * kg, 32 * (i >> 1) + col_t, lane);
        },
        [&](int h, u32x4(&f)[4]) {
#pragma unroll
          for (int i = 0; i < 4; ++i) dkacc[2 * h + (i >> 1)] = Tr::mfma(f[i], dsf[i & 1], dkacc[2 * h + (i >> 1)]);
        });
  }
}

// dK / dV with eight waves (two teams, as below) by workgroups that stay for the whole launch and walk one key
// block after the other without draining the pipeline of tiles in between.  A workgroup without tiles still costs
// 8 us (the chain header -> K / V fragments, records -> first tile, and at the end the sum over the wave pairs and
// the stores), a third of the time of a key block with 8 live pairs.  Here, while key block n is walked:
//   - the position of block n + 2 is drawn (one atomic add on the XCD's ticket counter by one lane; key rows are
//     handed out longest first, so a workgroup that drew a long one simply draws fewer);
//   - the header of block n + 1 is loaded (every wave its own copy);
//   - K and V of block n + 1 are copied into an LDS region (R) of their own, from which the fragments are read
//     when block n is done;
//   - the first tile of block n + 1 is copied into the free tile buffer during the last tile of block n.
// R also takes the partial sums of the wave pairs at the end of a block (after the next block's fragments have
// been read from it).  All conditions below are the same for the eight waves of a workgroup (they depend on headers
// and records only), so every wave passes the same barriers.
template <typename Tr, int NH, int NHV, bool DK, bool DV>
__device__ __forceinline__ void attn_bwd_kv8_walk(const bsa_attn_args &a, char *smem, int wave, int quad) {
  constexpr int kQRows = 0, kDoRows = NH * kBlockBytes, kStats = (NH + NHV) * kBlockBytes,
                kMask = kStats + kStatBytes;
  constexpr int kBufBytes = kMask + kSbs * kSbs;
  constexpr int kSlices = NH > NHV ? NH : NHV;
  constexpr int kTeamFloats = 2 * kSlices * 2 * 16 * 64;  // partial sums of one team
  char *region = smem + 2 * kBufBytes;                     // R: K / V of the next block, then the partial sums
  float *reduce_lds = reinterpret_cast<float *>(region) + (DK ? kTeamFloats : 0);
  int *mailbox = reinterpret_cast<int *>(region + 2 * kTeamFloats * 4);
  // P of the tile, handed from the dV team to the dK team: [quadrant][4][lane] of 16 bytes
  f32x4 *p_lds = reinterpret_cast<f32x4 *>(region + 2 * kTeamFloats * 4 + 64) + quad * 4 * 64 + (threadIdx.x & 63);

  const int tid = threadIdx.x, lane = tid & 63;
  const int li = lane & 31, kg = lane >> 5;
  const int wi = quad & 1, wj = quad >> 1;
  const int64_t rows = a.B * a.nk, chunk = (rows + 7) / 8;
  const int64_t first = (int64_t)(blockIdx.x & 7) * chunk;  // this XCD's eighth: positions first .. first + chunk - 1
  const BwdLists lists = bwd_lists(a);
  const int32_t *recs = reinterpret_cast<const int32_t *>(lists.query_rec);
  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  auto valid_ticket = [&](int t) { return t >= 0 && t < chunk && first + t < rows; };
  auto load_head = [&](int t) {
    int v = -1;
    if (valid_ticket(t) && lane < 16) v = lists.k_head[(first + t) * 16 + lane];
    return v;
  };
  auto draw = [&]() {  // one lane of the workgroup draws; -1 elsewhere
    int t = -1;
    if (tid == 0) t = atomicAdd(lists.kv_tickets + (blockIdx.x & 7), 1);
    return t;
  };

  // ---- the first block: nothing to overlap with
  int t_cur = (int)(blockIdx.x >> 3);
  if (!valid_ticket(t_cur)) return;  // same for the whole workgroup
  int drawn = draw();                // the position of the second block
  int head = load_head(t_cur);
  if (tid == 0) mailbox[0] = drawn;
  __syncthreads();
  int t_next = first_lane(mailbox[0]);
  __syncthreads();  // the mailbox may be written again

  u32x4 kfr[NH][4], vfr[NHV][4];
  {
#pragma unroll
    for (int h = 0; h < NH; ++h)
      load_resident(kfr[h], a.k, __builtin_amdgcn_readlane(head, 11 + h), a.n_k_blocks, 32 * wj + li, kg);
#pragma unroll
    for (int h = 0; h < NHV; ++h) {
      if constexpr (DK) load_resident(vfr[h], a.v, __builtin_amdgcn_readlane(head, 13 + h), a.n_v_blocks, 32 * wj + li, kg);
      else {
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) vfr[h][s4] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }
  f32x16 dkacc[DK ? NH * 2 : 1], dvacc[DV ? NHV * 2 : 1];
  auto clear = [&]() {
    if constexpr (DK) {
#pragma unroll
      for (int n = 0; n < NH * 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) dkacc[n][r] = 0.f;
    }
    if constexpr (DV) {
#pragma unroll
      for (int n = 0; n < NHV * 2; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) dvacc[n][r] = 0.f;
    }
  };
  clear();

  // registers of the tile in flight (the blocks themselves go straight to LDS)
  float stat = 0.f;  // thread 256 + t, t < 64: lse of query t; 320 + t: delta of query t
  // The record of the tile after next (field i in lanes i, 8 + i, ...), requested from inline assembly: between the
  // request and the wait in stage() nothing touches the register.
  int rec_in_flight = -1;
  const int32_t *const recs_lane = recs + (lane & 7);
  auto request_record = [&](int pos) {
    const int32_t *src = recs_lane + (int64_t)pos * 8;
    asm volatile("global_load_dword %0, %1, off" : "+v"(rec_in_flight) : "v"(src) : "memory");
  };
  int qb_nxt = 0, pm_nxt = -1, pb_nxt = -1, pair_nxt = 0;
  // requests the tile of record `rec` (field i in lane i) of batch entry `batch` into tile buffer `buf`
  auto fetch = [&](int rec, int buf, int64_t batch) {
    const int qb = __builtin_amdgcn_readlane(rec, 0);
    qb_nxt = qb;
    char *base = smem + first_lane(buf) * kBufBytes;  // the same for the whole wave: said so explicitly
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      const int pq = __builtin_amdgcn_readlane(rec, 1 + h);
      copy_block<8>(static_cast<const char *>(a.q) + (int64_t)(pq >= 0 ? pq : 0) * kBlockBytes, pq >= 0,
                    base + kQRows + h * kBlockBytes, wave, lane, tid);
    }
    // The dV team has the longer first half of a tile (S and P against dP): the dO blocks, the statistics and the
    // mask block are fetched by the dK team alone (waves 4 .. 7), the Q blocks by all eight waves.
    pm_nxt = __builtin_amdgcn_readlane(rec, 5);
    pb_nxt = __builtin_amdgcn_readlane(rec, 6);
    pair_nxt = __builtin_amdgcn_readlane(rec, 7);
    if (wave >= 4) {
#pragma unroll
      for (int h = 0; h < NHV; ++h) {
        const int po = __builtin_amdgcn_readlane(rec, 3 + h);
        copy_block<4>(static_cast<const char *>(a.d_o) + (int64_t)(po >= 0 ? po : 0) * kBlockBytes, po >= 0,
                      base + kDoRows + h * kBlockBytes, wave - 4, lane, tid - 256);
      }
      if (pm_nxt >= 0)
        copy_1k_to_lds(static_cast<const char *>(a.mask) + (int64_t)pm_nxt * (kSbs * kSbs) + (wave - 4) * 1024, lane * 16,
                       base + kMask + (wave - 4) * 1024);
    }
  };
  // The statistics of the tile of record `rec`: wave 4 requests the lse of its 64 queries, wave 5 their delta (the
  // other waves the lse as well, and drop it).  Requested from inline assembly like the copies: a load the compiler
  // knows of makes it wait for everything in flight (vmcnt(0)) at the next join, the copies included, which would
  // put the whole latency of the next tile in front of this tile's products.  Called on the straight path only (a
  // request in a branch of its own would let the compiler move the register at the join, with the load in flight);
  // when there is no next tile the value is not used: the record is then the last valid one, or the header of a next
  // key block without tiles, whose record fields are -1 (clamped: query block -1 of batch entry 0 would be a read in
  // front of the array).
  auto request_stat = [&](int rec, int64_t batch) {
    const int qb_of_rec = __builtin_amdgcn_readlane(rec, 0);
    const int64_t qrow = batch * a.nq + (qb_of_rec < 0 ? 0 : qb_of_rec);
    const float *src = (wave == 5 ? a.delta : a.lse) + qrow * kSbs + lane;
    asm volatile("global_load_dword %0, %1, off" : "+v"(stat) : "v"(src) : "memory");
  };
  // the statistics of the tile go to LDS through a register; then every copy of this wave has to have landed
  auto stage = [&](int buf) {
    char *base = smem + buf * kBufBytes;
    // everything this wave has requested has landed: its copies, the statistics, the record of the tile after
    // (the builtin, so that the compiler knows that nothing it has requested itself is pending either: a load it
    // believes to be in flight at the top of the loop makes it wait, with vmcnt(0), in front of the first product of
    // every tile, and that wait would include the copies of the next tile)
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" : "+v"(stat), "+v"(rec_in_flight) : : "memory");
    if (tid >= 256 && tid < 384)
      reinterpret_cast<float *>(base + kStats)[tid - 256] = (tid < 320 && stat == -INFINITY) ? INFINITY : stat;
  };
  // K and V of the block with header `h` into R
  auto prefetch_kv = [&](int h) {
#pragma unroll
    for (int s2 = 0; s2 < NH; ++s2) {
      const int pk = __builtin_amdgcn_readlane(h, 11 + s2);
      copy_block<8>(static_cast<const char *>(a.k) + (int64_t)(pk >= 0 ? pk : 0) * kBlockBytes, pk >= 0,
                    region + s2 * kBlockBytes, wave, lane, tid);
    }
#pragma unroll
    for (int s2 = 0; s2 < NHV; ++s2) {
      const int pv = __builtin_amdgcn_readlane(h, 13 + s2);
      copy_block<8>(static_cast<const char *>(a.v) + (int64_t)(pv >= 0 ? pv : 0) * kBlockBytes, pv >= 0,
                    region + (NH + s2) * kBlockBytes, wave, lane, tid);
    }
  };

  // dS of the tile before (dK team), kept in registers until the next tile has started: a store issued right
  // behind the tile's products would be waited for, with everything else in flight, at the end of that tile
  u32x4 ds_pending[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
  char *ds_pending_at = nullptr;
  auto store_pending_ds = [&]() {
    if constexpr (DK) {
      if (ds_pending_at) {
#pragma unroll
        // whole lines per instruction, read next by another kernel: past the caches (5 us less here, 5 in the dQ kernel)
        for (int u = 0; u < 2; ++u)
          __builtin_nontemporal_store(ds_pending[u], reinterpret_cast<u32x4 *>(ds_pending_at + 1024 * u));
        ds_pending_at = nullptr;
      }
    }
  };

  // the first block's fragments have arrived: from here on the compiler has no load of its own in flight when a
  // tile starts (see stage())
  __builtin_amdgcn_s_waitcnt(0x0F70);
  int buf = 0;            // the tile buffer of the current block's next tile
  bool staged = false;    // that tile has been requested and published already (during the block before)
  while (true) {
    buf = first_lane(buf);
    // ---- facts of the current block
    const uint32_t krow = (uint32_t)__builtin_amdgcn_readlane(head, 8), nk32 = (uint32_t)a.nk;  // int32 in the header
    const int64_t b = krow / nk32, kb = krow % nk32;
    const int q_begin = __builtin_amdgcn_readlane(head, 9), q_end = __builtin_amdgcn_readlane(head, 10);
    int seq_len = 0;
    if (causal) {
      const int64_t len = a.causal_lengths[b];
      seq_len = len < 0 ? 0 : (len > 0x7fffffffLL ? 0x7fffffff : (int)len);
    }
    const int kpos = (int)kb * kSbs + 32 * wj + li;
    const bool has_next = valid_ticket(t_next);
    // ---- for the blocks after this one: draw the position of the one after next, load the next header
    drawn = has_next ? draw() : -1;
    const int head_next = load_head(t_next);  // -1 in every lane when there is no next block
    int64_t b_next = 0;
    int q_begin_next = 0, q_end_next = 0;
    bool kv_requested = false;

    auto clamp_e = [&](int e) { return e < q_end ? e : q_end - 1; };

    if (q_begin < q_end) {
      // the record of the block's second tile: with the first tile staged during the block before, it was
      // requested (and waited for) there as well
      if (!staged) {
        request_record(clamp_e(q_begin + 1));
        fetch(head, buf, b);
        request_stat(head, b);
        stage(buf);  // waits for the two requests above inside this branch
        __syncthreads();
      }
      int rec = rec_in_flight;
      for (int e = q_begin; e < q_end; ++e) {
        const char *base = smem + buf * kBufBytes;
        const int qb = qb_nxt;
        const int64_t pm = pm_nxt, pb = pb_nxt;
        const int pair = pair_nxt;
        uint32_t mbits = 0;
        if (pm >= 0) {
          const uint8_t *mp = reinterpret_cast<const uint8_t *>(base + kMask) + (32 * wi + 4 * kg) * kSbs + 32 * wj + li;
#pragma unroll
          for (int r = 0; r < 16; ++r) mbits |= (uint32_t)mp[(8 * (r >> 2) + (r & 3)) * kSbs] << r;
        }
        const bool live = kv_quadrant_live(pm, mbits, causal, (int)kb, qb, seq_len, wi, wj);
        // the fragments the tile's first products start with: their latency lies behind the requests for the next tile
        u32x4 f0[4];
        kv_first_frags<NH, DK>(f0, base, wi, li, kg);
        const bool more = e + 1 < q_end;
        bool next_tile = more;
        if (e == q_begin + 1 && has_next) {
          // R is free (a barrier has passed since the partial sums of the block before were read) and the next
          // header has arrived (the wait at the end of the first tile covers its load)
          prefetch_kv(head_next);
          kv_requested = true;
        }
        // the next tile into the free buffer: the next one of this block, or (last tile) the first one of the next
        // block; one call for both, so that the copies are in the code once
        int rec_use = rec;
        int64_t batch_use = b;
        if (!more && has_next) {
          b_next = (uint32_t)__builtin_amdgcn_readlane(head_next, 8) / (uint32_t)a.nk;
          q_begin_next = __builtin_amdgcn_readlane(head_next, 9);
          q_end_next = __builtin_amdgcn_readlane(head_next, 10);
          next_tile = q_begin_next < q_end_next;
          rec_use = head_next;
          batch_use = b_next;
        }
        if (next_tile) fetch(rec_use, buf ^ 1, batch_use);
        request_stat(rec_use, batch_use);
        // the record of the tile after that one: of this block, or the second one of the next block
        request_record((!more && next_tile) ? (q_begin_next + 1 < q_end_next ? q_begin_next + 1 : q_end_next - 1)
                                            : clamp_e(e + 2));

        // dS of the tile before: behind the requests for the next tile, and with this whole tile to get there
        // before the next wait
        store_pending_ds();
        KvCarry carry;
        kv_first_half<Tr, NH, NHV, DK, DV>(carry, f0, live, a, base, qb, pm, pb, mbits, causal, seq_len, (int)kb, kpos,
                                           qk_scale, wi, wj, li, kg, lane, kfr, vfr, p_lds);
        __syncthreads();  // P is in LDS
        kv_second_half<Tr, NH, NHV, DK, DV>(carry, live, a, base, pb, wi, wj, li, kg, lane, dkacc, dvacc, p_lds, ds_pending);
        if constexpr (DK) {
          // dS of the pair for the dQ kernel, as the lanes hold it: quadrant (wi, wj) is 2 KiB, in it plane u (1 KiB)
          // holds ds_pending[u] of lane l at 16 l (see frag_ds)
          if (lists.ds) ds_pending_at = lists.ds + (int64_t)pair * kBlockBytes + (wi + 2 * wj) * 2048 + lane * 16;
        }

        if (next_tile) stage(buf ^ 1);
        else {  // K / V of the next block, the record
          __builtin_amdgcn_s_waitcnt(0x0F70);
          asm volatile("" : "+v"(rec_in_flight) : : "memory");
        }
        rec = rec_in_flight;
        __syncthreads();
        buf ^= 1;
        staged = next_tile && !more;
      }
    } else {
      staged = false;
    }

    // ---- end of the block
    store_pending_ds();
    if (has_next && !kv_requested) {
      // a block of fewer than two tiles: nothing was overlapped
      __syncthreads();  // R is free
      prefetch_kv(head_next);
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
    }
    // the stationary block's packed indices, before `head` is replaced
    int64_t pk[NH], pv[NHV];
#pragma unroll
    for (int h = 0; h < NH; ++h) pk[h] = __builtin_amdgcn_readlane(head, 11 + h);
#pragma unroll
    for (int h = 0; h < NHV; ++h) pv[h] = __builtin_amdgcn_readlane(head, 13 + h);
    if (has_next) {
      // the next block's fragments: this wave's keys j = 32 wj + li (every wave reads R; the first barrier of the
      // sum below ends these reads before R is written)
#pragma unroll
      for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) kfr[h][s4] = frag_rows(region + h * kBlockBytes, 32 * wj + li, 2 * s4 + kg);
      if constexpr (DK) {
#pragma unroll
        for (int h = 0; h < NHV; ++h)
#pragma unroll
          for (int s4 = 0; s4 < 4; ++s4) vfr[h][s4] = frag_rows(region + (NH + h) * kBlockBytes, 32 * wj + li, 2 * s4 + kg);
      }
    }
    if (tid == 0) mailbox[0] = drawn;  // published by the barriers of the sum
    // ---- add the two query halves, scale, store
    // wave wi keeps column half wi of every slice: it moves that half into the even accumulators
    if (wi == 1) {
      if constexpr (DK) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
          const f32x16 t = dkacc[2 * h];
          dkacc[2 * h] = dkacc[2 * h + 1];
          dkacc[2 * h + 1] = t;
        }
      }
      if constexpr (DV) {
#pragma unroll
        for (int h = 0; h < NHV; ++h) {
          const f32x16 t = dvacc[2 * h];
          dvacc[2 * h] = dvacc[2 * h + 1];
          dvacc[2 * h + 1] = t;
        }
      }
    }
    if constexpr (DK) exchange_odd_for_even(dkacc, reduce_lds, wi, wj, lane);
    if constexpr (DV) exchange_odd_for_even(dvacc, reduce_lds, wi, wj, lane);
    const int t_after = first_lane(mailbox[0]);
    // The sums leave as whole rows: every wave holds, for its key 32 wj + li, the column half db = wi of each slice
    // (register 4 q + t: column 32 db + 8 q + 4 kg + t, eight bytes of a row per lane) and writes it, rounded, into LDS, as rows of 128 bytes with the 16-byte chunks swizzled by the row, and all four waves of the
    // team store it from there, 16 rows each, eight lanes to a row: whole lines per instruction, past the caches.
    // (Stores of eight bytes per lane straight from the registers are written to memory as partial lines, twice
    // the bytes, and are waited for with the copies of the next tile.)
    {
      constexpr int kOut = DK ? NH : NHV;
      // in the tile buffer that the block's last tile has left free (the other one may hold the first tile of the
      // next block): the partial sums in R may still be read by the partner, and need no barrier of their own
      char *rows_lds = smem + first_lane(buf ^ 1) * kBufBytes + (DK ? 0 : NH * kBlockBytes);
      static_assert((NH + NHV) * kBlockBytes <= kBufBytes, "both teams' rows fit a tile buffer");
      {
        const int row = 32 * wj + li;
        const float factor = DK ? a.scale : 1.f;
#pragma unroll
        for (int h = 0; h < kOut; ++h)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x16 &acc = DK ? dkacc[DK ? 2 * h : 0] : dvacc[DV ? 2 * h : 0];  // column half wi
            u32x2 w;
            w[0] = Tr::pack2(acc[4 * q] * factor, acc[4 * q + 1] * factor);
            w[1] = Tr::pack2(acc[4 * q + 2] * factor, acc[4 * q + 3] * factor);
            *reinterpret_cast<u32x2 *>(rows_lds + h * kBlockBytes + row * 128 + (((4 * wi + q) ^ (row & 7)) << 4) + 8 * kg) = w;
          }
      }
      __syncthreads();
#pragma unroll
      for (int h = 0; h < kOut; ++h) {
        const int64_t p = DK ? pk[DK ? h : 0] : pv[DV ? h : 0];
        if (p < 0) continue;
        char *out = static_cast<char *>(DK ? a.dk : a.dv) + p * kBlockBytes;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int r = 16 * quad + 8 * i + (lane >> 3), c = lane & 7;
          const u32x4 v = *reinterpret_cast<const u32x4 *>(rows_lds + h * kBlockBytes + r * 128 + ((c ^ (r & 7)) << 4));
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + r * 128 + c * 16));
        }
      }
    }
    if (!has_next) break;
    clear();
    head = head_next;
    t_cur = t_next;
    t_next = t_after;
    __syncthreads();  // the mailbox and the partial sums have been read
  }
}

// Eight waves: waves 0 .. 3 accumulate dV, waves 4 .. 7 dK and dBias, two waves per SIMD.  Each team fits 256
// registers per lane, which the two sets of accumulators in one wave do not; the tile is fetched once for both.
constexpr int kKv8Threads = 512;
template <typename Tr, int NH, int NHV>
__global__ __launch_bounds__(kKv8Threads, 1) void attn_bwd_kv8_walk_kernel(bsa_attn_args a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int wave = first_lane((int)threadIdx.x >> 6);
  if (wave < 4) attn_bwd_kv8_walk<Tr, NH, NHV, false, true>(a, smem, wave, wave & 3);
  else attn_bwd_kv8_walk<Tr, NH, NHV, true, false>(a, smem, wave, wave & 3);
}

// ---------------------------------------------------------------------------------------------------------
// dQ of one query block
template <typename Tr, int NH, int NHV>
__global__ __launch_bounds__(kBwdThreads, 2) void attn_bwd_q_kernel(bsa_attn_args a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int kKRows = 0, kVRows = NH * kBlockBytes;
  constexpr int kBufBytes = (NH + NHV) * kBlockBytes;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = first_lane(tid >> 6);
  const int li = lane & 31, kg = lane >> 5;
  const int wi = wave & 1, wj = wave >> 1;
  const int64_t qpos_in_order = xcd_row();
  const BwdLists lists = bwd_lists(a);
  // the dK / dV kernel that follows hands out key rows by tickets: the workgroups of an XCD start with the
  // positions 0 .. slots - 1 of its eighth, the next one to hand out is `slots`
  if (blockIdx.x == 0 && tid < 8) lists.kv_tickets[tid] = (int32_t)kv_slots(a.B * a.nk);
  if (qpos_in_order >= a.B * a.nq) return;
  // the workgroup's header, int i in lane i (lanes 0 .. 7 double as the record of the first tile)
  int head = -1;
  if (lane < 16) head = lists.q_head[qpos_in_order * 16 + lane];
  const int64_t qrow = __builtin_amdgcn_readlane(head, 8);
  const int64_t b = qrow / a.nq, qb = qrow % a.nq;

  int64_t pq[NH];
  bool any = false;
#pragma unroll
  for (int h = 0; h < NH; ++h) {
    pq[h] = __builtin_amdgcn_readlane(head, 11 + h);
    any = any || pq[h] >= 0;
  }

  // this wave's queries: B operands Q[i][.], dO[i][.] with i = 32 wi + li
  const int qi = 32 * wi + li;
  u32x4 qfr[NH][4], dofr[NHV][4];
#pragma unroll
  for (int h = 0; h < NHV; ++h) load_resident(dofr[h], a.d_o, __builtin_amdgcn_readlane(head, 13 + h), a.n_o_blocks, qi, kg);
#pragma unroll
  for (int h = 0; h < NH; ++h) load_resident(qfr[h], a.q, pq[h], a.n_q_blocks, qi, kg);
  // a query without any visible key has lse = -inf and P = 0 everywhere: +inf gives exp2(s - lse) = 0 for it
  const float lse_raw = a.lse[qrow * kSbs + qi];
  const float lse = lse_raw == -INFINITY ? INFINITY : lse_raw;
  // delta[i] = sum over the output slices of rowsum(o * dO) of the wave's queries, from the dO fragments it holds
  // anyway and the same pieces of o: the two lanes of a query hold every other 16-byte piece of its rows.  The
  // dK / dV kernel, which runs after this one, reads it from a.delta; it needs it for every row that has a pair,
  // with or without a q block, so this comes before the test below.  Both key halves compute the same bits; the
  // first writes them.
  float delta = 0.f;
  {
    u32x4 ofr[NHV][4];
#pragma unroll
    for (int h = 0; h < NHV; ++h) load_resident(ofr[h], a.o, __builtin_amdgcn_readlane(head, 13 + h), a.n_o_blocks, qi, kg);
#pragma unroll
    for (int h = 0; h < NHV; ++h)
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4)
#pragma unroll
        for (int t = 0; t < 4; ++t) delta = Tr::dot2(ofr[h][s4][t], dofr[h][s4][t], delta);
    delta = sum_across32(delta);
    if (wj == 0 && kg == 0) a.delta[qrow * kSbs + qi] = delta;
  }
  if (!any) return;

  f32x16 dqacc[NH * 2];
#pragma unroll
  for (int n = 0; n < NH * 2; ++n)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[n][r] = 0.f;

  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  int seq_len = 0;
  if (causal) {
    const int64_t len = a.causal_lengths[b];
    seq_len = len < 0 ? 0 : (len > 0x7fffffffLL ? 0x7fffffff : (int)len);
  }
  const int qpos = (int)qb * kSbs + qi;

  const int k_begin = __builtin_amdgcn_readlane(head, 9), k_end = __builtin_amdgcn_readlane(head, 10);
  if (k_begin < k_end) {
    // the record of a list entry, field i in lane i: one 32-byte load, two tiles before the tile is used
    const int32_t *recs = reinterpret_cast<const int32_t *>(lists.key_rec);
    auto load_record = [&](int pos) -> int {
      int v = -1;
      if (lane < 8) v = recs[(int64_t)pos * 8 + lane];
      return v;
    };
    auto clamp_e = [&](int e) { return e < k_end ? e : k_end - 1; };

    uint32_t mask_w[4];  // mask bytes of keys 32 wj + 8 q + 4 kg .. + 3 of this lane's query, one word per q
    u32x2 bias_w[4];     // bias elements likewise
    int kb_nxt, pm_nxt, pb_nxt;

    auto fetch = [&](int rec, int buf) {
      kb_nxt = __builtin_amdgcn_readlane(rec, 0);
      char *base = smem + buf * kBufBytes;
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        const int pk = __builtin_amdgcn_readlane(rec, 1 + h);
        copy_block(static_cast<const char *>(a.k) + (int64_t)(pk >= 0 ? pk : 0) * kBlockBytes, pk >= 0,
                   base + kKRows + h * kBlockBytes, wave, lane, tid);
      }
#pragma unroll
      for (int h = 0; h < NHV; ++h) {
        const int pv = __builtin_amdgcn_readlane(rec, 3 + h);
        copy_block(static_cast<const char *>(a.v) + (int64_t)(pv >= 0 ? pv : 0) * kBlockBytes, pv >= 0,
                   base + kVRows + h * kBlockBytes, wave, lane, tid);
      }
      pm_nxt = __builtin_amdgcn_readlane(rec, 5);
      pb_nxt = __builtin_amdgcn_readlane(rec, 6);
      if (pm_nxt >= 0) {
        const char *mp = static_cast<const char *>(a.mask) + (int64_t)pm_nxt * (kSbs * kSbs);
        const uint32_t off = (uint32_t)qi * 64u + 32u * wj + 4u * kg;
#pragma unroll
        for (int q = 0; q < 4; ++q) mask_w[q] = *reinterpret_cast<const uint32_t *>(mp + off + 8 * q);
      }
      if (pb_nxt >= 0) {
        const char *bp = static_cast<const char *>(a.bias) + (int64_t)pb_nxt * kBlockBytes;
        const uint32_t off = (uint32_t)qi * 128u + 64u * wj + 8u * kg;
#pragma unroll
        for (int q = 0; q < 4; ++q) bias_w[q] = *reinterpret_cast<const u32x2 *>(bp + off + 16 * q);
      }
    };
    // every copy of this wave has to have landed before the barrier
    auto stage = [&](int) { __builtin_amdgcn_s_waitcnt(0x0F70); };

    int rec;
    {
      rec = load_record(clamp_e(k_begin + 1));
      fetch(head, 0);
      stage(0);
      __syncthreads();
    }

    for (int e = k_begin; e < k_end; ++e) {
      const int buf = (e - k_begin) & 1;
      const char *base = smem + buf * kBufBytes;
      const int kb = kb_nxt;
      const int64_t pm = pm_nxt, pb = pb_nxt;
      uint32_t mask_c[4];
      u32x2 bias_c[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) mask_c[q] = mask_w[q];
      if (pb >= 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) bias_c[q] = bias_w[q];
      }
      const bool more = e + 1 < k_end;
      if (more) fetch(rec, buf ^ 1);
      rec = load_record(clamp_e(e + 2));

      bool live = true;
      if (pm >= 0) live = !__all((mask_c[0] & mask_c[1] & mask_c[2] & mask_c[3]) == 0x01010101u);
      if (causal) {
        const int k_first = kb * kSbs + 32 * wj, q_first = (int)qb * kSbs + 32 * wi;
        if (k_first > q_first + 31 || q_first >= seq_len || k_first >= seq_len) live = false;
      }
      if (live) {
        // ---- S^T and dP^T of this wave's quadrant: lane owns query qi, register r key 32 wj + 8 (r / 4) + 4 kg + r % 4 ----
        f32x16 sacc, dpacc;
  #pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] = dpacc[r] = 0.f;
        staged_products<NH + NHV>(
            [&](int k, u32x4(&f)[4]) {
              const char *src = base + (k < NH ? kKRows + k * kBlockBytes : kVRows + (k - NH) * kBlockBytes);
  #pragma unroll
              for (int s = 0; s < 4; ++s) f[s] = frag_rows(src, 32 * wj + li, 2 * s + kg);
            },
            [&](int k, u32x4(&f)[4]) {
  #pragma unroll
              for (int s = 0; s < 4; ++s) {
                if (k < NH) sacc = Tr::mfma(f[s], qfr[k < NH ? k : 0][s], sacc);
                else dpacc = Tr::mfma(f[s], dofr[k < NH ? 0 : k - NH][s], dpacc);
              }
            });

        float ds[16];
        // the plain path: no bias, no mask block, causal predicate true for every score of the quadrant
        auto gradients = [&](auto plain_tag) {
          constexpr bool kPlain = decltype(plain_tag)::value;
  #pragma unroll
          for (int q = 0; q < 4; ++q)
  #pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int r = 4 * q + t;
              float s = sacc[r] * qk_scale;
              if constexpr (!kPlain) {
                if (pb >= 0) {
                  const uint32_t bw = bias_c[q][t >> 1];
                  s = s + Tr::widen((uint16_t)((t & 1) ? (bw >> 16) : (bw & 0xffffu))) * kLog2e;
                }
                if (causal) {
                  const int kpos = kb * kSbs + 32 * wj + 8 * q + 4 * kg + t;
                  s = (kpos > qpos || qpos >= seq_len || kpos >= seq_len) ? -INFINITY : s;
                }
                if (pm >= 0) s = ((mask_c[q] >> (8 * t)) & 0xffu) ? -INFINITY : s;
              }
              const float p = __builtin_amdgcn_exp2f(s - lse);
              ds[r] = p * (dpacc[r] - delta);
            }
        };
        bool plain = pb < 0 && pm < 0;
        if (causal) {
          const int k_last = kb * kSbs + 32 * wj + 31, q_first = (int)qb * kSbs + 32 * wi;
          plain = plain && k_last <= q_first && q_first + 31 < seq_len;
        }
        if (plain) gradients(std::true_type{});
        else gradients(std::false_type{});
        u32x4 dsf[2];
  #pragma unroll
        for (int u = 0; u < 2; ++u)
  #pragma unroll
          for (int t = 0; t < 4; ++t) dsf[u][t] = Tr::pack2(ds[8 * u + 2 * t], ds[8 * u + 2 * t + 1]);

        // ---- dQ^T += K^T dS^T over this wave's 32 keys ----
        const int col_t = 16 * ((lane >> 4) & 1);
        staged_products<NH>(
            [&](int h, u32x4(&f)[4]) {
  #pragma unroll
              for (int i = 0; i < 4; ++i)
                f[i] = frag_cols_t(base + kKRows + h * kBlockBytes, 32 * wj + 16 * (i & 1) + 4 * kg, 32 * (i >> 1) + col_t, lane);
            },
            [&](int h, u32x4(&f)[4]) {
  #pragma unroll
              for (int i = 0; i < 4; ++i) dqacc[2 * h + (i >> 1)] = Tr::mfma(f[i], dsf[i & 1], dqacc[2 * h + (i >> 1)]);
            });

      }  // live

      if (more) stage(buf ^ 1);
      __syncthreads();
    }
  }

  // ---- add the two key halves, scale, store ----
  reduce_partner(dqacc, reinterpret_cast<float *>(smem), wj == 1, wi, lane);
  if (wj == 1) return;
  // The wave's 32 rounded rows pass through LDS behind the partial sums (rows of 128 bytes, chunks swizzled by the
  // row) and leave as whole lines, eight lanes to a row, past the caches; rows and chunks are the wave's own: no
  // barrier.
  char *rows_lds = smem + NH * 2 * 2 * 16 * 64 * 4;
  static_assert(NH * 2 * 2 * 16 * 64 * 4 + NH * kBlockBytes <= 2 * kBufBytes, "the rows fit behind the partial sums");
#pragma unroll
  for (int h = 0; h < NH; ++h)
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x16 &acc = dqacc[2 * h + db];
        u32x2 w;
        w[0] = Tr::pack2(acc[4 * q] * a.scale, acc[4 * q + 1] * a.scale);
        w[1] = Tr::pack2(acc[4 * q + 2] * a.scale, acc[4 * q + 3] * a.scale);
        *reinterpret_cast<u32x2 *>(rows_lds + h * kBlockBytes + qi * 128 + (((4 * db + q) ^ (qi & 7)) << 4) + 8 * kg) = w;
      }
#pragma unroll
  for (int h = 0; h < NH; ++h) {
    if (pq[h] < 0) continue;
    char *out = static_cast<char *>(a.dq) + pq[h] * kBlockBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 32 * wi + 8 * i + (lane >> 3), c = lane & 7;
      const u32x4 v = *reinterpret_cast<const u32x4 *>(rows_lds + h * kBlockBytes + r * 128 + ((c ^ (r & 7)) << 4));
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + r * 128 + c * 16));
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Second operand of dQ^T += K^T dS^T from a dS block as the dK / dV kernel leaves it: quadrant (wi, wj) of the pair
// (queries 32 wi .., keys 32 wj ..) is 2 KiB; in it, plane u (1 KiB) holds at 16 l the eight values of lane l =
// 32 kg + key % 32 of that kernel: dS of key l % 32 and queries 32 wi + 16 u + 8 h + 4 kg + t for h = 0, 1 and
// t = 0 .. 3.  Seen as rows of 16 values (both planes of a lane side by side), row 32 g + j holds key j and the
// sixteen queries 8 (c / 4) + 4 g + c % 4, c = 0 .. 15.  The transposing load hands lane i of a 16-lane group column
// i of four rows: with group g16 of a wave half on the rows of g = g16, the 32 lanes of a half cover the quadrant's
// 32 queries, lane (i, g16) holding query 8 (i / 4) + 4 g16 + i % 4 (query_of_lane) and keys key0 .. + 3 and
// key0 + 8 .. + 11, the same eight as frag_cols_t gives for the first operand.
__device__ static inline u32x4 frag_ds(const char *blob, int wi, int wj, int key0, int lane) {
  const int s = lane & 15, g16 = (lane >> 4) & 1;
  const int row = 32 * g16 + key0 + (s >> 2);
  const char *p0 = blob + (wi + 2 * wj) * 2048 + ((s & 3) >> 1) * 1024 + row * 16 + (s & 1) * 8;
  const char *p1 = p0 + 8 * 16;
  const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)p0);
  const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)p1);
  const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
  return u32x4{l2[0], l2[1], h2[0], h2[1]};
}
// copy_2k_to_lds for data that is read once: past the caches (the dS blocks of the dQ kernel: 190 -> 184 us)
__device__ static inline void copy_2k_to_lds_nt(const char *base, uint32_t off, char *dst) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr_t)dst;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024 nt"
               :
               : "v"(off), "s"(base), "s"(lds_addr)
               : "memory");
}

__device__ static inline int query_of_lane(int lane) { return 8 * ((lane & 15) >> 2) + 4 * ((lane >> 4) & 1) + (lane & 3); }

// dQ of one query block from the dS blocks the dK / dV kernel has written: dQ^T += K^T dS^T, one product per pair
// and no scores.  Wave (wi, wj) owns queries 32 wi .. + 31 (in the order of query_of_lane) and the head-dimension
// columns 32 NH wj .. + 32 NH - 1 (slice wj with two slices, half of the slice with one) and contracts over all 64
// keys of every tile, so no wave needs another's sums.  The dS block of the e-th pair of the list is block e of
// the scratch region (the records are numbered that way), so its address needs no record.  A tile is the K slices
// and the dS block of a pair, 8 KiB each, copied asynchronously into LDS; there is ONE buffer for the K slices
// (their copies are requested when the products of the tile before are done, and waited for) and two for dS
// (the block of the next tile, which comes from memory, is requested one tile ahead).  What hides the latency of
// the copies is the number of workgroups per compute unit that the small buffers allow, each at another point of
// its list.  The kernel's time is that of its memory traffic: on configuration 4 of the benchmark it reads 0.55 GB
// of dS and 0.13 GB of K from memory and writes 0.13 GB of dQ in 195 microseconds (4.4 TB/s; the same with dS
// from the L2: 135; without the products: 192; without the copies: 70), and every arrangement of the copies
// measured ends there: two buffers for the whole tile and three workgroups per compute unit 215; a ring of five
// dS blocks with two waves copying dS and two K, two workgroups, 238; one buffer, five workgroups, 198; with the
// second dS buffer 195; the tile through registers (loads one tile ahead, written to LDS by the waves) 194.
// Every pair of the list is
// multiplied: quadrants without a surviving score hold zeros.
constexpr int kDqWorkgroupsPerCu = 5;
template <typename Tr, int NH>
__global__ __launch_bounds__(kBwdThreads, kDqWorkgroupsPerCu) void attn_bwd_dq_kernel(bsa_attn_args a) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int kDsRows = NH * kBlockBytes;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = first_lane(tid >> 6);
  const int kg = lane >> 5;
  const int wi = wave & 1, wj = wave >> 1;
  const int64_t qpos_in_order = xcd_row();
  const BwdLists lists = bwd_lists(a);
  if (qpos_in_order >= a.B * a.nq) return;
  int head = -1;
  if (lane < 16) head = lists.q_head[qpos_in_order * 16 + lane];
  // this wave's NH column blocks of 32: block n is columns 32 (NH wj + n) of the head dimension, that is slice
  // (NH wj + n) / 2, half (NH wj + n) % 2
  const int first_block = NH * wj;
  bool any = false;
#pragma unroll
  for (int h = 0; h < NH; ++h) any = any || __builtin_amdgcn_readlane(head, 11 + h) >= 0;
  if (!any) return;

  f32x16 dqacc[NH];
#pragma unroll
  for (int n = 0; n < NH; ++n)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[n][r] = 0.f;

  const int k_begin = __builtin_amdgcn_readlane(head, 9), k_end = __builtin_amdgcn_readlane(head, 10);
  if (k_begin < k_end) {
    const int32_t *recs = reinterpret_cast<const int32_t *>(lists.key_rec);
    // eight records at a time, field f of the j-th in lane 8 j + f (two lines of the list, which come from memory:
    // requested eight tiles before their first use)
    auto load_records = [&](int first) -> int {
      int pos = first + (lane >> 3);
      pos = pos < k_end ? pos : k_end - 1;
      return recs[(int64_t)pos * 8 + (lane & 7)];
    };
    // the K slices of the tile of record j of `chunk`, a quarter of every block per wave, into the one K buffer
    auto fetch_k = [&](int chunk, int j) {
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        const int pk = __builtin_amdgcn_readlane(chunk, 8 * j + 1 + h);
        copy_block(static_cast<const char *>(a.k) + (int64_t)(pk >= 0 ? pk : 0) * kBlockBytes, pk >= 0,
                   smem + h * kBlockBytes, wave, lane, tid);
      }
    };
    // the dS block of list entry e (it comes from memory: one tile ahead, into the other of two buffers)
    auto fetch_ds = [&](int e) {
      copy_2k_to_lds_nt(lists.ds + (int64_t)e * kBlockBytes + wave * 2048, lane * 16,
                        smem + kDsRows + first_lane((e - k_begin) & 1) * kBlockBytes + wave * 2048);
    };

    const int col_t = 16 * ((lane >> 4) & 1);
    int chunk = load_records(k_begin), chunk_next = chunk;
    fetch_ds(k_begin);
    for (int e = k_begin; e < k_end; ++e) {
      const int j = (e - k_begin) & 7;
      if (j == 0 && e != k_begin) chunk = chunk_next;
      // the header holds the first record, so the first tile does not wait for the list
      if (e == k_begin) fetch_k(head, 0);
      else fetch_k(chunk, j);
      // this tile's copies have landed; the next tile's dS block (two loads, the youngest) may stay in flight
      if (e + 1 < k_end) {
        fetch_ds(e + 1);
        __builtin_amdgcn_s_waitcnt(0x0F72);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      __syncthreads();
      // the next eight records: in flight behind this tile's products
      if (j == 0 && e + 8 < k_end) chunk_next = load_records(e + 8);
      const char *ds_tile = smem + kDsRows + ((e - k_begin) & 1) * kBlockBytes;

      // dS^T as the second operand: query 32 wi + query_of_lane, keys 16 u + 4 kg .. + 3 and + 8 .. + 11
      u32x4 dsf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) dsf[u] = frag_ds(ds_tile, wi, u >> 1, 16 * (u & 1) + 4 * kg, lane);
      // stage n: column block first_block + n of K^T against all four key steps
      staged_products<NH>(
          [&](int n, u32x4(&f)[4]) {
            const int blk = first_block + n;
#pragma unroll
            for (int u = 0; u < 4; ++u)
              f[u] = frag_cols_t(smem + (blk >> 1) * kBlockBytes, 16 * u + 4 * kg, 32 * (blk & 1) + col_t, lane);
          },
          [&](int n, u32x4(&f)[4]) {
#pragma unroll
            for (int u = 0; u < 4; ++u) dqacc[n] = Tr::mfma(f[u], dsf[u], dqacc[n]);
          });
      __syncthreads();  // the buffer is free
    }
  }

  // ---- scale, round, store.  Register 4 q + t of block n is column 32 (first_block + n) + 8 q + 4 kg + t of the
  // lane's query: eight bytes of a row at a time.  The rounded block goes through LDS (rows of 128 bytes, chunks
  // swizzled by the row; the tile buffers are free) and leaves as whole rows, 16 per wave, eight lanes to a row,
  // past the caches: half the bytes written of stores straight from the registers. ----
  const int qi = 32 * wi + query_of_lane(lane);
#pragma unroll
  for (int n = 0; n < NH; ++n) {
    const int blk = first_block + n;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const f32x16 &acc = dqacc[n];
      u32x2 w;
      w[0] = Tr::pack2(acc[4 * q] * a.scale, acc[4 * q + 1] * a.scale);
      w[1] = Tr::pack2(acc[4 * q + 2] * a.scale, acc[4 * q + 3] * a.scale);
      *reinterpret_cast<u32x2 *>(smem + (blk >> 1) * kBlockBytes + qi * 128 + (((4 * (blk & 1) + q) ^ (qi & 7)) << 4) + 8 * kg) = w;
    }
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < NH; ++h) {
    const int64_t pq = __builtin_amdgcn_readlane(head, 11 + h);
    if (pq < 0) continue;
    char *out = static_cast<char *>(a.dq) + pq * kBlockBytes;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = 16 * wave + 8 * i + (lane >> 3), c = lane & 7;
      const u32x4 v = *reinterpret_cast<const u32x4 *>(smem + h * kBlockBytes + r * 128 + ((c ^ (r & 7)) << 4));
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + r * 128 + c * 16));
    }
  }
}

__global__ void fill_zero_f32_kernel(float *p, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = 0.f;
}

// The kernels that ask for more than 64 KiB of LDS say so once per process and device: the attribute belongs to
// the loaded code object of a device, so the calls are made the first time a launch runs on it.
constexpr int kMaxDevices = 64;
template <typename Tr, int NH, int NHV>
int set_lds_attributes(int lds_q, int lds_walk, int lds_dq) {
  static std::atomic<bool> done[kMaxDevices];
  int dev = 0;
  BSA_HIP(hipGetDevice(&dev));
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && done[dev].load(std::memory_order_acquire)) return BSA_OK;
  BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_bwd_q_kernel<Tr, NH, NHV>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_q));
  BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_bwd_kv8_walk_kernel<Tr, NH, NHV>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_walk));
  BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_bwd_dq_kernel<Tr, NH>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_dq));
  if (tracked) done[dev].store(true, std::memory_order_release);
  return BSA_OK;
}

__global__ void fill_zero_u32x4_kernel(u32x4 *p, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = u32x4{0u, 0u, 0u, 0u};
}

int zero_blocks(void *p, int64_t n_blocks, hipStream_t s) {
  if (n_blocks <= 0 || p == nullptr) return BSA_OK;
  const int64_t n = n_blocks * (kBlockBytes / 16);
  int64_t blocks = cdiv(n, 1024);
  if (blocks > 65536) blocks = 65536;
  fill_zero_u32x4_kernel<<<(unsigned)blocks, 256, 0, s>>>(static_cast<u32x4 *>(p), n);
  return check_launch("fill_zero_u32x4_kernel");
}

template <typename Tr, int NH, int NHV>
int launch_bwd(const bsa_attn_args &a, hipStream_t s) {
  const int64_t qrows = a.B * a.nq, krows = a.B * a.nk;
  if (a.dbias && a.n_bias_blocks > 0) {
    // bias blocks outside the attention layout get no gradient
    const int64_t n = a.n_bias_blocks * kSbs * kSbs;
    int64_t blocks = cdiv(n, 1024);
    if (blocks > 65536) blocks = 65536;
    fill_zero_f32_kernel<<<(unsigned)blocks, 256, 0, s>>>(a.dbias, n);
    if (int rc = check_launch("fill_zero_f32_kernel")) return rc;
  }
  if (qrows == 0 || krows == 0) {
    // no query or no key: no pair, every gradient is zero (the walk's tickets are set by the kernels of the query
    // side, which have nothing to launch here)
    if (int rc = zero_blocks(a.dq, a.n_q_blocks, s)) return rc;
    if (int rc = zero_blocks(a.dk, a.n_k_blocks, s)) return rc;
    return zero_blocks(a.dv, a.n_v_blocks, s);
  }
  constexpr int lds_q = 2 * (NH + NHV) * kBlockBytes;
  // tile buffers, the region of the next block's K / V and of the partial sums of both teams, the mailbox, P of a tile
  constexpr int kSlices = NH > NHV ? NH : NHV;
  constexpr int lds_walk = 2 * ((NH + NHV) * kBlockBytes + kStatBytes + kSbs * kSbs) + 2 * (2 * kSlices * 2 * 16 * 64) * 4 +
                           64 + 4 * 4 * 64 * 16;
  static_assert((NH + NHV) * kBlockBytes <= 2 * (2 * kSlices * 2 * 16 * 64) * 4, "K and V fit the region");
  constexpr int lds_dq = (NH + 2) * kBlockBytes;
  if (int rc = set_lds_attributes<Tr, NH, NHV>(lds_q, lds_walk, lds_dq)) return rc;
  if (!a.bwd_scratch_ready) {
    const BwdLists L = bwd_lists(a);
    if (a.mask != nullptr && a.n_mask_blocks > 0) {
      attn_bwd_mask_dead_kernel<<<(unsigned)cdiv(a.n_mask_blocks, 4), kBwdThreads, 0, s>>>(
          static_cast<const u32x4 *>(a.mask), L.mask_dead, a.n_mask_blocks);
      if (int rc = check_launch("attn_bwd_mask_dead_kernel")) return rc;
    }
    attn_bwd_records_kernel<<<(unsigned)cdiv(qrows, 4), kBwdThreads, 0, s>>>(a, false);
    if (int rc = check_launch("attn_bwd_records_kernel")) return rc;
    attn_bwd_records_kernel<<<(unsigned)cdiv(krows, 4), kBwdThreads, 0, s>>>(a, true);
    if (int rc = check_launch("attn_bwd_records_kernel")) return rc;
    attn_bwd_order_kernel<<<16, kOrderThreads, 0, s>>>(a);
    if (int rc = check_launch("attn_bwd_order_kernel")) return rc;
  }
  // With room for the dS blocks: delta and the tickets first, then the dK / dV walk, which leaves dS^T of every pair
  // behind, then dQ = dS K as a product of its own.  Without: the dQ kernel forms the scores and dS of its pairs a
  // second time; it runs first and leaves delta and the tickets for the walk.
  const bool from_ds = bwd_lists(a).ds != nullptr;
  if (from_ds) {
    attn_bwd_delta_kernel<Tr><<<(unsigned)qrows, kBwdThreads, 0, s>>>(a);
    if (int rc = check_launch("attn_bwd_delta_kernel")) return rc;
  } else {
    attn_bwd_q_kernel<Tr, NH, NHV><<<(unsigned)(cdiv(qrows, 8) * 8), kBwdThreads, lds_q, s>>>(a);
    if (int rc = check_launch("attn_bwd_q_kernel")) return rc;
  }
  attn_bwd_kv8_walk_kernel<Tr, NH, NHV><<<(unsigned)(kv_slots(krows) * 8), kKv8Threads, lds_walk, s>>>(a);
  if (int rc = check_launch("attn_bwd_kv8_walk_kernel")) return rc;
  if (from_ds) {
    attn_bwd_dq_kernel<Tr, NH><<<(unsigned)(cdiv(qrows, 8) * 8), kBwdThreads, lds_dq, s>>>(a);
    if (int rc = check_launch("attn_bwd_dq_kernel")) return rc;
  }
  return BSA_OK;
}

template <typename Tr>
int dispatch_bwd(const bsa_attn_args &a, hipStream_t s) {
  if (a.nh == 1 && a.nhv == 1) return launch_bwd<Tr, 1, 1>(a, s);
  if (a.nh == 2 && a.nhv == 2) return launch_bwd<Tr, 2, 2>(a, s);
  if (a.nh == 1 && a.nhv == 2) return launch_bwd<Tr, 1, 2>(a, s);
  if (a.nh == 2 && a.nhv == 1) return launch_bwd<Tr, 2, 1>(a, s);
  return 1;
}

}  // namespace

int attn_mask_dead(const void *mask, int64_t n_mask_blocks, uint8_t *dead, hipStream_t s) {
  attn_bwd_mask_dead_kernel<<<(unsigned)cdiv(n_mask_blocks, 4), kBwdThreads, 0, s>>>(static_cast<const u32x4 *>(mask),
                                                                                     dead, n_mask_blocks);
  return check_launch("attn_bwd_mask_dead_kernel");
}

size_t attn_bwd_scratch_bytes(int64_t B, int64_t nq, int64_t nk, int64_t n_layout_blocks, int64_t n_mask_blocks) {
  return bwd_lists_bytes(B, nq, nk, n_layout_blocks, n_mask_blocks);
}

size_t attn_bwd_ds_bytes(int64_t n_layout_blocks) { return (size_t)n_layout_blocks * kBlockBytes; }

int attn_bwd_mfma(const bsa_attn_args &a, hipStream_t s) {
  if (a.sbs != kSbs || (a.dtype != BSA_BF16 && a.dtype != BSA_F16)) return 1;
  if ((a.B * a.nq > 0 && a.key_indices == nullptr) || (a.B * a.nk > 0 && a.query_indices == nullptr)) return 1;
  if (a.bwd_scratch == nullptr) return 1;  // the matrix-core kernels walk the records built in the scratch
  return a.dtype == BSA_BF16 ? dispatch_bwd<MBf16>(a, s) : dispatch_bwd<MF16>(a, s);
}

}  // namespace bsa
