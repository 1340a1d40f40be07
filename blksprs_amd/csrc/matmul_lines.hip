// Line kernel of the block-sparse GEMM for the two backward products (16-bit operands, sbs == 64):
//   dX = dO Y^T  (blksprs/ops/matmul.py:135-139): a line is a block row (b, i) of dX;
//   dY = X^T dO  (blksprs/ops/matmul.py:141-145): a line is a block column (b, j) of dY.
// In both, one operand has a whole line of blocks that every output block of the line needs (row i resp. column j
// of dO: the STREAMED operand), and the other one block per (output block, streamed block) pair (Y(k, j) resp.
// X(i, k): the PRIVATE operand).  A line of dO is some 60 blocks on a product layout, four times what LDS holds,
// so unlike the forward product's x row it cannot stay resident: it streams through a ring in LDS, once, while
// the accumulators of the line's output blocks stay in registers for the whole line.  dO is then read from
// memory once per launch, where a kernel that takes output blocks one by one fetches it once per output block.
//
// Work: one workgroup of 8 waves per part of a line = up to 16 of its output blocks; wave w owns the part's
// blocks w and w + 8 (two 64 x 64 accumulators, 128 registers) and walks the streamed blocks in order; where the
// private operand has a block for one of its output blocks there is a pair: the private block is copied
// (asynchronously, global -> LDS) into the wave's own 8 KiB stage, its operand fragments are read into
// registers, the stage is handed to the copy of the next pair's block at once, and 16 matrix-core products
// follow with the streamed operand's fragments read from the ring.  Which pairs exist is found from the reverse
// indices of the three layouts with one lane per streamed block: no lists are built for this kernel.
//
// The ring: kRing slots of 8 KiB.  The waves do not move in step (a wave has a pair at one streamed block in four
// on a layout of 25 % density), so a barrier per block would make every block as slow as the slowest wave.
// Instead LDS holds, per slot, `ready` = 1 + the streamed block it holds, written by the wave that copied it once
// its copy has landed, and per wave `pos` = the lowest streamed block the wave still needs.  Streamed block d is
// copied by wave d % 8, as soon as all eight waves have moved past block d - kRing and that block has been announced; a
// wave checks for its copying duty between pairs and while it waits for a block.  No wave waits for anything but
// a wave of its own workgroup that is either computing or in the same loop, so the protocol cannot stall: the
// lowest block not yet copied is always the next duty of some wave, and the waves that have not released its
// slot are at blocks below it, which are there.  Every wait is bounded all the same: a wave that polls 2^22 times
// sets `broken`, after which every wait gives up and the workgroup runs to its end (with wrong results; a test
// would see them, the GPU does not hang).
//
// Contraction index: dX contracts the columns of both blocks (row fragments, 128-bit LDS reads); dY contracts
// the rows of both (the transposing LDS read).  Both operands lie in LDS row-major with the 16-byte chunks of a
// row swizzled (t_swizzle), which is conflict-free for either read.  The product is formed transposed, as in the
// row kernel, and a finished block leaves through the wave's stage as whole rows (rows_flush).
#include "attn_mfma_common.h"
#include "mfma_tile_out.h"

namespace {

using namespace bsa::mfma;

constexpr int kWaves = 8;
constexpr int kRing = 11;
constexpr int kMaxLine = 512;  // blocks of a line that the lists in LDS hold
constexpr int kSlotsPerPart = 2 * kWaves;
constexpr int kSpinLimit = 1 << 22;

struct LinesLds {
  char ring[kRing][kBlockBytes];
  char stage[kWaves][kBlockBytes];
  int32_t s_idx[kMaxLine];    // packed index of the d-th streamed block of the line
  int32_t s_coord[kMaxLine];  // its position along the line
  int32_t count_s[kWaves], count_o[kWaves];  // candidates that wave w found active
  int32_t o_idx[kSlotsPerPart], o_coord[kSlotsPerPart];
  int32_t ready[kRing];  // 1 + the streamed block the slot holds, once its copy has landed
  int32_t pos[kWaves];   // wave w needs no streamed block below pos[w] any more
  int32_t broken;
};
constexpr int kLinesLds = sizeof(LinesLds);
static_assert(kMaxLine == 64 * kWaves, "one chunk of candidates per wave");
static_assert(kLinesLds <= 160 * 1024, "fits the LDS of a compute unit");

__device__ __forceinline__ int lds_peek(int32_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// one 8 KiB block, global -> LDS, by one wave: 8 asynchronous copies of 1 KiB (8 rows), chunks swizzled by the row
__device__ __forceinline__ void copy_block_by_wave(const char *blk, char *dst, int lane) {
  const uint32_t lane_off = (lane >> 3) * 128 + (((lane & 7) ^ t_swizzle(lane >> 3)) << 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) copy_2k_to_lds(blk + i * 2048, lane_off, dst + i * 2048);
}

// The same for a block that is read once per launch (a block of the streamed operand): with the nontemporal hint,
// so that it does not push the private operand's blocks, which are read again and again, out of the L2.
__device__ __forceinline__ void copy_block_by_wave_once(const char *blk, char *dst, int lane) {
  const uint32_t lane_off = (lane >> 3) * 128 + (((lane & 7) ^ t_swizzle(lane >> 3)) << 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr_t)(dst + i * 2048);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt\n\tglobal_load_lds_dwordx4 %0, %1 offset:1024 nt"
                 :
                 : "v"(lane_off), "s"(blk + i * 2048), "s"(lds_addr)
                 : "memory");
  }
}

struct LinesArgs {
  const char *s, *p;
  char *out;
  const int64_t *pidx_s, *pidx_p, *pidx_o;
  const int32_t *part_table;  // [0]: number of parts; [1 + position]: line << 6 | part, in the order of the launch
  int64_t n_lines, lines_per_batch;
  int64_t n_s, n_o;  // candidate positions of a line: streamed blocks, output blocks
  // position of candidate t of line (b, l) in pidx_s: b s_sb + l s_sl + t s_st; likewise pidx_o with u; the private
  // block of (output candidate u, streamed candidate t) of batch entry b: pidx_p[b p_sb + u p_su + t p_st]
  int64_t s_sb, s_sl, s_st, o_sb, o_sl, o_su, p_sb, p_su, p_st;
  int64_t nnz_s, nnz_p, nnz_out;
  int32_t *error;  // NULL, or 32 ints: [0] = 1 once a wait ran out, then what the first such wave saw
};

// Parts per line: ceil(active output candidates / 16), in two classes: parts of more than 8 output blocks (some
// wave owns two: a long part) and the others (a short part: at most the last part of a line); one wave per line.
__global__ __launch_bounds__(256) void lines_count_kernel(LinesArgs a, int32_t *long_parts, int32_t *short_parts) {
  const int64_t line = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 6;
  if (line >= a.n_lines) return;
  const int lane = threadIdx.x & 63;
  const int64_t b = line / a.lines_per_batch, l = line % a.lines_per_batch;
  int n = 0;
  for (int64_t u0 = 0; u0 < a.n_o; u0 += 64) {
    const int64_t u = u0 + lane;
    int64_t v = -1;
    if (u < a.n_o) v = a.pidx_o[b * a.o_sb + l * a.o_sl + u * a.o_su];
    n += __popcll(__ballot(v >= 0 && v < a.nnz_out));
  }
  if (lane == 0) {
    const int rest = n % kSlotsPerPart;
    long_parts[line] = n / kSlotsPerPart + (rest > kWaves ? 1 : 0);
    short_parts[line] = rest > 0 && rest <= kWaves ? 1 : 0;
  }
}

// The table of parts.  The parts of a batch entry are consecutive; inside a batch entry all long parts come
// first, then all short ones, each group in the order of the lines: workgroups that run side by side then have
// about the same amount of work, start and end together, and walk the streamed operand's positions together, so
// that the blocks of the private operand they share are in the L2 when the second one asks.  long_before /
// short_before: exclusive prefix sums over the lines (with the totals at [n_lines]).  One thread per line.
__global__ __launch_bounds__(256) void lines_table_kernel(LinesArgs a, const int32_t *long_before,
                                                          const int32_t *short_before, int32_t *table) {
  const int64_t line = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (line == 0) table[0] = long_before[a.n_lines] + short_before[a.n_lines];
  if (line >= a.n_lines) return;
  const int64_t first = line - line % a.lines_per_batch, end = first + a.lines_per_batch;
  const int batch_base = long_before[first] + short_before[first];
  const int n_long = long_before[line + 1] - long_before[line], n_short = short_before[line + 1] - short_before[line];
  for (int p = 0; p < n_long; ++p) table[1 + batch_base + (long_before[line] - long_before[first]) + p] = (int32_t)(line << 6) | p;
  if (n_short)
    table[1 + batch_base + (long_before[end] - long_before[first]) + (short_before[line] - short_before[first])] =
        (int32_t)(line << 6) | n_long;
}

// exclusive prefix sums of counts[0 .. n) into offsets[0 .. n], one workgroup
__global__ __launch_bounds__(1024) void lines_scan_kernel(const int32_t *counts, int32_t *offsets, int64_t n) {
  __shared__ int wave_sum[16];
  __shared__ int carry;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int64_t base = 0; base < n; base += 1024) {
    const int64_t i = base + tid;
    const int v = i < n ? counts[i] : 0;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int t = __shfl_up(incl, d);
      if (lane >= d) incl += t;
    }
    if (lane == 63) wave_sum[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += wave_sum[w];
    if (i < n) offsets[i] = before + incl - v;
    __syncthreads();
    if (tid == 1023) carry = before + incl;
    __syncthreads();
  }
  if (tid == 0) offsets[n] = carry;
}

template <typename Tr, bool TR>
__global__ __launch_bounds__(kWaves * 64, 1) void matmul_lines_kernel(LinesArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char lines_smem[];
  LinesLds &L = *reinterpret_cast<LinesLds *>(lines_smem);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = first_lane(tid >> 6);
  const int li = lane & 31, kg = lane >> 5;

  // ---- which part of which line: every XCD takes a contiguous eighth of the table, in order
  const int64_t total = a.part_table[0];
  const int64_t chunk = (total + 7) / 8;
  const int64_t at = (int64_t)(blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
  if ((int64_t)(blockIdx.x >> 3) >= chunk || at >= total) return;
  const int32_t entry = a.part_table[1 + at];
  const int64_t line = entry >> 6;
  const int part = entry & 63;
  if (line < 0 || line >= a.n_lines) return;  // a corrupt table must not turn into a wild read
  const int64_t b = line / a.lines_per_batch, l = line % a.lines_per_batch;

  if (tid < kRing) L.ready[tid] = 0;
  if (tid < kWaves) L.pos[tid] = 0;
  if (tid == 0) L.broken = 0;

  // ---- the line's streamed blocks and the part's output blocks, compacted into LDS.  A line has at most 512
  // candidates of either kind: wave w looks at candidates 64 w .. 64 w + 63 of both (the two loads are in flight
  // together), the counts meet in LDS, and every wave writes its entries behind those of the waves before it.
  int64_t vs = -1, vo = -1;
  const int64_t t = (int64_t)wave * 64 + lane;
  if (t < a.n_s) vs = a.pidx_s[b * a.s_sb + l * a.s_sl + t * a.s_st];
  if (t < a.n_o) vo = a.pidx_o[b * a.o_sb + l * a.o_sl + t * a.o_su];
  if (vs >= a.nnz_s) vs = -1;
  if (vo >= a.nnz_out) vo = -1;
  const unsigned long long votes_s = __ballot(vs >= 0), votes_o = __ballot(vo >= 0);
  if (lane == 0) {
    L.count_s[wave] = __popcll(votes_s);
    L.count_o[wave] = __popcll(votes_o);
  }
  if (tid < kSlotsPerPart) L.o_idx[tid] = -1;
  __syncthreads();
  int n_streamed = 0;
  {
    int before_s = 0, before_o = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) {
      const int cs = L.count_s[i], co = L.count_o[i];
      n_streamed += cs;
      before_s += i < wave ? cs : 0;
      before_o += i < wave ? co : 0;
    }
    if (vs >= 0) {
      const int rank = before_s + __popcll(votes_s & ((1ull << lane) - 1));
      L.s_idx[rank] = (int32_t)vs;
      L.s_coord[rank] = (int32_t)t;
    }
    const int slot = before_o + __popcll(votes_o & ((1ull << lane) - 1)) - part * kSlotsPerPart;
    if (vo >= 0 && slot >= 0 && slot < kSlotsPerPart) {
      L.o_idx[slot] = (int32_t)vo;
      L.o_coord[slot] = (int32_t)t;
    }
  }
  n_streamed = first_lane(n_streamed);
  __syncthreads();

  // this wave's output blocks
  const int n_segments = (n_streamed + 63) >> 6;
  int o_idx[2], o_coord[2];
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    o_idx[x] = first_lane(L.o_idx[wave + kWaves * x]);
    o_coord[x] = first_lane(L.o_coord[wave + kWaves * x]);
  }

  f32x16 acc[2][2][2];  // [output block][column half][row half]
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[x][i][j][r] = 0.f;

  char *stage = L.stage[wave];

  // ---- copying duty: streamed blocks wave, wave + 8, ...
  int duty = wave;          // the next block this wave copies
  int duty_inflight = -1;   // the block whose copies are on their way
  bool duty_is_young = false;  // those copies were requested after this wave's last copy of a private block
  int dbg_where = 0, dbg_d = -1;
  auto spin_ok = [&](int &spins) {
    if (++spins > kSpinLimit) {
      if (a.error != nullptr && lane == 0 && atomicCAS(a.error, 0, 1) == 0) {
        int32_t *e = a.error;
        e[1] = wave; e[2] = dbg_where; e[3] = dbg_d; e[4] = duty; e[5] = duty_inflight; e[6] = n_streamed;
        e[7] = (int)blockIdx.x;
        for (int i = 0; i < kWaves; ++i) e[8 + i] = L.pos[i];
        for (int i = 0; i < 10; ++i) e[16 + i] = L.ready[i];
        e[26] = (int)line; e[27] = part; e[28] = o_idx[0]; e[29] = o_idx[1];
      }
      L.broken = 1;
    }
    return lds_peek(&L.broken) == 0;
  };
  // the copies of duty_inflight have landed (the caller has waited): say so
  auto duty_publish = [&]() {
    if (duty_inflight >= 0) {
      // LDS executes a wave's instructions in order and the caller's wait stands in front of this store: a plain
      // store (a release would make the compiler wait for every copy in flight, the next pair's block included)
      asm volatile("" ::: "memory");
      __hip_atomic_store(&L.ready[duty_inflight % kRing], duty_inflight + 1, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_WORKGROUP);
      duty_inflight = -1;
    }
  };
  // One LDS read per lane tells what a wave wants to know between two pairs: the eight waves' positions (lanes
  // 0 .. 7), what the slot of its next duty block holds (lane 8) and what the slot of streamed block d holds (the
  // other lanes).  The duty block is requested if no copy of this wave is in flight, every wave has moved past the
  // block that its slot held, and that block's copy has landed and been announced (a block that no wave has a pair
  // with is passed by all before its copy is there: a later announcement would overwrite this block's, and its data
  // could land on top of this block's).  Returns whether block d is there.
  auto poll = [&](int d) {
    int32_t *at_lane = lane < kWaves ? &L.pos[lane] : &L.ready[(lane == kWaves ? duty : d) % kRing];
    const int v = lds_peek(at_lane);
    const bool have = __builtin_amdgcn_readlane(v, kWaves + 1) == d + 1;
    if (duty_inflight < 0 && duty < n_streamed) {
      const bool passed = __all(lane >= kWaves || v > duty - kRing);
      if (passed && (duty < kRing || __builtin_amdgcn_readlane(v, kWaves) == duty - kRing + 1)) {
        const int32_t blk = first_lane(L.s_idx[duty]);
        copy_block_by_wave_once(a.s + (int64_t)blk * kBlockBytes, L.ring[duty % kRing], lane);
        duty_inflight = duty;
        duty_is_young = true;
        duty += kWaves;
      }
    }
    return have;
  };

  // ---- the walk over this wave's pairs.  Segment g = streamed blocks 64 g .. 64 g + 63, lane e looks up the
  // private block of (its output blocks, streamed block 64 g + e).
  int seg = -1;
  unsigned long long todo[2] = {0ull, 0ull};  // pairs of the segment not yet handed out, per output block
  int pv[2] = {-1, -1};                       // lane e: private block of the pair (x, 64 seg + e)
  auto load_segment = [&](int g) {
    seg = g;
    const int d = 64 * g + lane;
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      int64_t v = -1;
      if (d < n_streamed && o_idx[x] >= 0)
        v = a.pidx_p[b * a.p_sb + (int64_t)o_coord[x] * a.p_su + (int64_t)L.s_coord[d] * a.p_st];
      if (v >= a.nnz_p) v = -1;
      pv[x] = (int)v;
      todo[x] = __ballot(v >= 0);
    }
  };
  struct Pair {
    int d, x, priv;  // streamed block, output block of this wave, private block; d < 0: none left
  };
  auto next_pair = [&]() {
    Pair p{-1, 0, 0};
    while (true) {
      const unsigned long long any = todo[0] | todo[1];
      if (any) {
        const int e = __builtin_ctzll(any);
        const int x = (todo[0] >> e) & 1 ? 0 : 1;
        todo[x] &= ~(1ull << e);
        p.d = 64 * seg + e;
        p.x = x;
        p.priv = __builtin_amdgcn_readlane(x == 0 ? pv[0] : pv[1], e);
        return p;
      }
      if (seg + 1 >= n_segments) return p;
      load_segment(seg + 1);
    }
  };

  // This wave needs no streamed block below d any more.  Its reads of those blocks were issued before this store
  // and LDS executes a wave's instructions in order; the statement in front keeps the compiler from moving them.
  auto release_to = [&](int d) {
    asm volatile("" ::: "memory");
    __hip_atomic_store(&L.pos[wave], d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  };

  poll(0);  // the first duty block: its copy is on its way while the first pairs are looked up
  Pair cur = next_pair();
  if (cur.d >= 0) copy_block_by_wave(a.p + (int64_t)cur.priv * kBlockBytes, stage, lane);
  duty_is_young = false;

  auto multiply = [&](f32x16 (&c)[2][2], const u32x4 (&pf)[4][2], const char *sb) {
    // the streamed operand's fragments of step s + 1 are requested before the products of step s, and no further
    // ahead (the scheduling barriers: with all eight reads hoisted to the top an accumulator is spilled)
    u32x4 sf[2][2];
    auto read_s = [&](int s, u32x4 (&f)[2]) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if constexpr (TR) f[h] = frag_cols_t(sb, 16 * s + 4 * kg, 32 * h + 16 * ((lane >> 4) & 1), lane);
        else f[h] = *reinterpret_cast<const u32x4 *>(sb + (32 * h + li) * 128 + (((2 * s + kg) ^ t_swizzle(li)) << 4));
      }
    };
    read_s(0, sf[0]);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (s + 1 < 4) read_s(s + 1, sf[(s + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          // A: the operand whose free index is the output column, B: the output row
          if constexpr (TR) c[bj][bi] = Tr::mfma(sf[s & 1][bj], pf[s][bi], c[bj][bi]);
          else c[bj][bi] = Tr::mfma(pf[s][bj], sf[s & 1][bi], c[bj][bi]);
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // one pair, added to the accumulators `c` of its output block
  auto do_pair = [&](f32x16 (&c)[2][2]) {
    release_to(cur.d);
    const Pair nxt = next_pair();
    // the private block of this pair has landed: only a duty's 8 copies can be younger
    if (duty_inflight >= 0 && duty_is_young) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    u32x4 pf[4][2];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if constexpr (TR) pf[s][h] = frag_cols_t(stage, 16 * s + 4 * kg, 32 * h + 16 * ((lane >> 4) & 1), lane);
        else pf[s][h] = *reinterpret_cast<const u32x4 *>(stage + (32 * h + li) * 128 + (((2 * s + kg) ^ t_swizzle(li)) << 4));
      }
    // every read of the stage has returned before the next block is copied over it
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int h = 0; h < 2; ++h) asm volatile("" : "+v"(pf[s][h]));
    const bool more = nxt.d >= 0;
    if (more) copy_block_by_wave(a.p + (int64_t)nxt.priv * kBlockBytes, stage, lane);
    duty_is_young = false;
    // the duty requested a pair ago is older than those 8 copies
    if (duty_inflight >= 0) {
      if (more) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      duty_publish();
    }
    // the streamed block of this pair
    {
      int spins = 0;
      dbg_where = 1; dbg_d = cur.d;
      while (!poll(cur.d) && spin_ok(spins)) {
        __builtin_amdgcn_s_sleep(2);
        if (duty_inflight >= 0) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          duty_publish();
        }
      }
      asm volatile("" ::: "memory");  // the block's fragments are read after the flag
    }
    multiply(c, pf, L.ring[cur.d % kRing]);
    cur = nxt;
  };
  // Runs of pairs of one output block, each run a loop of its own that touches one set of accumulators only (one
  // loop with a test per pair makes the compiler carry both sets through copies: 64 moves per pair and spills).
  while (cur.d >= 0) {
    while (cur.d >= 0 && cur.x == 0) do_pair(acc[0]);
    while (cur.d >= 0 && cur.x == 1) do_pair(acc[1]);
  }
  // no pair left: every streamed block is released, and this wave's remaining duties are done as their slots come free
  release_to(n_streamed);
  {
    int spins = 0;
    dbg_where = 2;
    while ((duty < n_streamed || duty_inflight >= 0) && spin_ok(spins)) {
      if (duty_inflight >= 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        duty_publish();
      }
      poll(0);
      if (duty_inflight < 0) __builtin_amdgcn_s_sleep(2);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }

  // ---- the wave's output blocks, through its own stage
#pragma unroll
  for (int x = 0; x < 2; ++x)
    if (o_idx[x] >= 0) rows_flush<Tr>(acc[x], a.out + (int64_t)o_idx[x] * kBlockBytes, stage, lane);
}

template <typename Tr>
int launch_lines(const LinesArgs &a, int64_t max_parts, int contract_rows, hipStream_t s) {
  static bool configured = false;  // raising the dynamic LDS limit is per function, once per process
  if (!configured) {
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&matmul_lines_kernel<Tr, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLinesLds));
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&matmul_lines_kernel<Tr, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLinesLds));
    configured = true;
  }
  const unsigned grid = (unsigned)(bsa::cdiv(max_parts, 8) * 8);
  if (contract_rows) matmul_lines_kernel<Tr, true><<<grid, kWaves * 64, kLinesLds, s>>>(a);
  else matmul_lines_kernel<Tr, false><<<grid, kWaves * 64, kLinesLds, s>>>(a);
  return bsa::check_launch("matmul_lines_kernel");
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int fill_args(const char *who, LinesArgs &a, const bsa_lines_args *in) {
  BSA_REQUIRE(in != nullptr, "%s: NULL argument block", who);
  BSA_REQUIRE(in->n_batches >= 0 && in->lines_per_batch >= 0 && in->n_streamed >= 0 && in->n_outputs >= 0,
              "%s: negative layout size", who);
  BSA_REQUIRE(in->nnz_streamed >= 0 && in->nnz_private >= 0 && in->nnz_out >= 0, "%s: negative block count", who);
  BSA_REQUIRE(in->nnz_streamed < 0x7fffffffLL && in->nnz_private < 0x7fffffffLL && in->nnz_out < 0x7fffffffLL,
              "%s: too many blocks", who);
  BSA_REQUIRE(in->n_batches * in->lines_per_batch < 0x7fffffffLL, "%s: too many lines", who);
  BSA_REQUIRE(in->n_streamed <= kMaxLine, "%s: a line of at most %d streamed blocks (got %lld)", who, kMaxLine,
              (long long)in->n_streamed);
  BSA_REQUIRE(in->n_outputs <= kMaxLine, "%s: a line of at most %d output blocks (got %lld)", who, kMaxLine,
              (long long)in->n_outputs);
  a.s = static_cast<const char *>(in->streamed);
  a.p = static_cast<const char *>(in->priv);
  a.out = static_cast<char *>(in->out);
  a.pidx_s = in->pidx_streamed;
  a.pidx_p = in->pidx_private;
  a.pidx_o = in->pidx_out;
  a.part_table = in->part_table;
  a.n_lines = in->n_batches * in->lines_per_batch;
  a.lines_per_batch = in->lines_per_batch;
  a.n_s = in->n_streamed;
  a.n_o = in->n_outputs;
  a.s_sb = in->streamed_strides[0], a.s_sl = in->streamed_strides[1], a.s_st = in->streamed_strides[2];
  a.o_sb = in->out_strides[0], a.o_sl = in->out_strides[1], a.o_su = in->out_strides[2];
  a.p_sb = in->private_strides[0], a.p_su = in->private_strides[1], a.p_st = in->private_strides[2];
  a.nnz_s = in->nnz_streamed, a.nnz_p = in->nnz_private, a.nnz_out = in->nnz_out;
  a.error = in->error;
  return BSA_OK;
}

}  // namespace

extern "C" int bsa_matmul_lines_parts(const bsa_lines_args *args, int32_t *scratch, int32_t *part_table,
                                      bsa_stream_t stream) {
  const char *who = "bsa_matmul_lines_parts";
  LinesArgs a;
  if (int rc = fill_args(who, a, args)) return rc;
  BSA_REQUIRE(part_table != nullptr && scratch != nullptr, "%s: NULL pointer", who);
  BSA_REQUIRE(a.n_lines < (1 << 25), "%s: too many lines for a table entry", who);
  hipStream_t s = bsa::as_stream(stream);
  // scratch: parts per line in the two classes, then their prefix sums
  int32_t *long_parts = scratch, *short_parts = scratch + a.n_lines;
  int32_t *long_before = scratch + 2 * a.n_lines, *short_before = long_before + a.n_lines + 1;
  if (a.n_lines > 0) {
    BSA_REQUIRE(a.pidx_o != nullptr, "%s: NULL pidx_out", who);
    lines_count_kernel<<<(unsigned)bsa::cdiv(a.n_lines, 4), 256, 0, s>>>(a, long_parts, short_parts);
    if (int rc = bsa::check_launch("lines_count_kernel")) return rc;
  }
  lines_scan_kernel<<<1, 1024, 0, s>>>(long_parts, long_before, a.n_lines);
  if (int rc = bsa::check_launch("lines_scan_kernel")) return rc;
  lines_scan_kernel<<<1, 1024, 0, s>>>(short_parts, short_before, a.n_lines);
  if (int rc = bsa::check_launch("lines_scan_kernel")) return rc;
  lines_table_kernel<<<(unsigned)bsa::cdiv(a.n_lines + 1, 256), 256, 0, s>>>(a, long_before, short_before, part_table);
  return bsa::check_launch("lines_table_kernel");
}

extern "C" int bsa_matmul_lines(const bsa_lines_args *args, int contract_rows, int sbs, int dtype,
                                bsa_stream_t stream) {
  const char *who = "bsa_matmul_lines";
  LinesArgs a;
  if (int rc = fill_args(who, a, args)) return rc;
  BSA_REQUIRE(sbs == 64, "%s: sbs must be 64 (got %d)", who, sbs);
  BSA_REQUIRE(dtype == BSA_F16 || dtype == BSA_BF16, "%s: dtype must be fp16 or bf16 (got %d)", who, dtype);
  if (a.nnz_out == 0 || a.n_lines == 0) return BSA_OK;
  BSA_REQUIRE(a.out && a.pidx_s && a.pidx_p && a.pidx_o && a.part_table, "%s: NULL pointer", who);
  BSA_REQUIRE(aligned16(a.s) && aligned16(a.p) && aligned16(a.out), "%s: buffers must be 16-byte aligned", who);
  // every line with an output block has ceil(blocks / 16) parts: at most nnz_out / 16 + n_lines in all
  const int64_t max_parts = a.nnz_out / kSlotsPerPart + a.n_lines;
  BSA_REQUIRE(max_parts < 0x7ffffff0LL, "%s: too many parts", who);
  hipStream_t s = bsa::as_stream(stream);
  if (dtype == BSA_BF16) return launch_lines<MBf16>(a, max_parts, contract_rows, s);
  return launch_lines<MF16>(a, max_parts, contract_rows, s);
}
