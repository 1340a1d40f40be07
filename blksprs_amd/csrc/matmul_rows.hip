// Row kernel of the block-sparse GEMM (16-bit operands, sbs == 64, untransposed operands): one workgroup of
// 8 waves owns one part of a block row (b, i) of the output, at most 64 output blocks.
//
// x: the row's x blocks are consecutive in memory; up to 18 of them (144 KiB) are copied once into LDS by
// asynchronous global -> LDS copies and stay there while the waves walk the row's output blocks, so x is
// read from L2 once per row, and a wave never waits for x.  x blocks beyond the 18 resident ones are read
// from global memory in fragment layout (slow path, rare).
//
// Work split: the part's output blocks are dealt to the 8 waves in ascending order, each to the wave that has
// the least work so far (list scheduling over the blocks' numbers of (x, y) pairs, done once per layout by
// bsa_matmul_rows_records, which leaves one 64-bit mask of blocks per wave in the row's record).  The waves
// therefore move through the row's columns together: the y blocks in flight on a compute unit, and on the XCD
// whose rows belong to one batch entry, lie in a narrow band of columns, and the waves of a workgroup end within
// a block of each other.  Rows are handed to workgroups in the order the caller gives (longest first keeps the
// tail of the launch short).
//
// y: only y blocks stream.  A wave walks the pairs of its blocks as one flat sequence.  Which pair comes next
// is scalar work that runs a pair ahead of everything else: the list entry of the next pair and the pair range
// of the next block are requested (scalar loads) while the current entry is turned into addresses, so no load
// of metadata is waited for.  Each y block travels global -> registers -> LDS -> matrix-core operand: two
// register slots of 8 KiB hold the y blocks of the next two pairs, so a block is requested about one and a half
// pairs before it is used.  The loads are issued from inline assembly and waited for with hand-placed
// s_waitcnt vmcnt(n): the compiler would join the outstanding loads with vmcnt(0) at every branch.  vmcnt
// counts vector memory instructions in issue order, so "all but the youngest n" is exact as long as n is not
// larger than the number of instructions issued after the loads waited for; every n used below is such a lower
// bound (the other slot's 8 loads, plus the 8 stores of an output block written since).
//
// Per pair, per quarter of the contraction (16 k): 2 KiB of the y block are written to the wave's LDS stage
// as stored (k rows), and read back with the transposing LDS load, which delivers the matrix-core operand
// whose contraction index runs over rows; the x operand is a 128-bit row read from the panel.  LDS executes
// one wave's instructions in order, so stage writes and reads of consecutive quarters are queued back to
// back without waits in between; only the fragment registers bound the depth.  The loop is software pipelined
// across pairs (the first half of the next pair is staged while the second half of this one is multiplied).
//
// The product is formed transposed (y fragments as the A operand, x fragments as B), which leaves 4
// consecutive output columns of one row in each lane; a finished block is rounded, passed through the stage
// 16 rows at a time and written with 16-byte stores that cover whole rows.  Output blocks without any pair are
// written (zeros) before the walk starts.
#include "attn_mfma_common.h"
#include "mfma_tile_out.h"

namespace {

using namespace bsa::mfma;

constexpr int kPanelCap = 18;
constexpr int kWaves = 8;
constexpr int kStageBytes = 2048;                                   // 16 rows of 128 bytes
constexpr int kRowsLds = kPanelCap * 8192 + kWaves * kStageBytes;  // 160 KiB

struct YSlot {
  u32x4 v[8];  // v[i] = rows 8 i + lane / 8, chunk lane % 8 of one 64 x 64 block
};

// requests the 8 KiB block at yb into the slot; lane_lo = 16 * lane, lane_hi = lane_lo + 4096.  The address
// arrives in scalar registers that a vector instruction (v_readlane) may have written just before: a vector
// memory instruction must not read such a register within the next 5 wait states, and the compiler does not
// look into inline assembly, so the wait states are spelled out here.
__device__ __forceinline__ void y_issue(YSlot &s, const char *yb, uint32_t lane_lo, uint32_t lane_hi) {
  asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2" : "=v"(s.v[0]) : "v"(lane_lo), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(s.v[1]) : "v"(lane_lo), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:2048" : "=v"(s.v[2]) : "v"(lane_lo), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:3072" : "=v"(s.v[3]) : "v"(lane_lo), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(s.v[4]) : "v"(lane_hi), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(s.v[5]) : "v"(lane_hi), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:2048" : "=v"(s.v[6]) : "v"(lane_hi), "s"(yb) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:3072" : "=v"(s.v[7]) : "v"(lane_hi), "s"(yb) : "memory");
}

// waits until at most N vector memory instructions are outstanding; the slot's registers pass through the
// statement so that no use of them can be moved in front of it
#define BSA_Y_WAIT(slot_, n_)                                                                                  \
  asm volatile("s_waitcnt vmcnt(" #n_ ")"                                                                      \
               : "+v"((slot_).v[0]), "+v"((slot_).v[1]), "+v"((slot_).v[2]), "+v"((slot_).v[3]),               \
                 "+v"((slot_).v[4]), "+v"((slot_).v[5]), "+v"((slot_).v[6]), "+v"((slot_).v[7])                \
               :                                                                                               \
               : "memory")

// no instruction: the slot's registers pass through the statement, so that no use of them can be moved in
// front of the wait that precedes it
#define BSA_Y_TIE(slot_)                                                                                       \
  asm volatile(""                                                                                              \
               : "+v"((slot_).v[0]), "+v"((slot_).v[1]), "+v"((slot_).v[2]), "+v"((slot_).v[3]),               \
                 "+v"((slot_).v[4]), "+v"((slot_).v[5]), "+v"((slot_).v[6]), "+v"((slot_).v[7])                \
               :                                                                                               \
               : "memory")

// XOR applied to the 16-byte chunk index of row r of a y quarter in the stage.  A transposing read serves 32
// lanes at a time: rows r .. r + 3 (r a multiple of 4), 64 consecutive bytes of each.  Two 128-byte rows span
// the 64 banks once, so rows r and r + 2 must put their 64 bytes into different halves of the row.
__device__ __forceinline__ int y_swizzle(int r) { return ((r >> 1) & 1) << 2; }

__device__ __forceinline__ u32x2 read_tr(const char *p) {
  const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)p);
  return __builtin_bit_cast(u32x2, v);
}

// per-lane LDS addresses that do not change during the kernel
struct LaneAddr {
  char *wr[2];      // stage write: rows lane / 8 and 8 + lane / 8 of a quarter, chunk lane % 8
  const char *tr[2][2];  // transposing reads: [column block][rows k0 .. k0 + 3 | k0 + 4 .. k0 + 7]
  uint32_t xoff[4];  // x fragment of k step s inside a panel block (row lane % 32; the second row block is + 4096)
};

// operand fragments of one quarter (16 k) of a pair: [column block] of y, [row block] of x
struct Frags {
  u32x4 fy[2], fx[2];
};

// where the x block of a pair is read from: its swizzled copy in the panel, or (not resident: rare) global
// memory; all wave uniform
struct XSource {
  const char *lds;
  int px;  // packed index of the x block (range checked), for the read from global memory
  bool resident;
};

// Writes quarter S (k = 16 S .. 16 S + 15) of the y block in the slot to the stage and reads the quarter's
// operand fragments: y with transposing reads from the stage, x with 128-bit row reads from the panel.
template <int S>
__device__ __forceinline__ void stage_and_read(Frags &f, const YSlot &ys, const XSource &xs, const LaneAddr &la,
                                               const char *x, int lane) {
  *reinterpret_cast<u32x4 *>(la.wr[0]) = ys.v[2 * S];
  *reinterpret_cast<u32x4 *>(la.wr[1]) = ys.v[2 * S + 1];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const u32x2 lo = read_tr(la.tr[b][0]), hi = read_tr(la.tr[b][1]);
    f.fy[b] = u32x4{lo[0], lo[1], hi[0], hi[1]};
    f.fx[b] = *reinterpret_cast<const u32x4 *>(xs.lds + la.xoff[S] + 4096 * b);
  }
  if (!xs.resident) {
    // rare: only the fragments pass through the branch (not the accumulators), and they are used inside it,
    // which puts the wait for these loads here and not in front of the multiplications of every pair
    const int li = lane & 31, kg = lane >> 5;
    const char *xglob = x + (int64_t)xs.px * 8192;
#pragma unroll
    for (int b = 0; b < 2; ++b)
      f.fx[b] = *reinterpret_cast<const u32x4 *>(xglob + (uint32_t)((32 * b + li) * 128 + (2 * S + kg) * 16));
    asm volatile("" : "+v"(f.fx[0]), "+v"(f.fx[1]));
  }
}

template <typename Tr>
__device__ __forceinline__ void multiply(f32x16 (&acc)[2][2], const Frags &f) {
#pragma unroll
  for (int bj = 0; bj < 2; ++bj)
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) acc[bj][bi] = Tr::mfma(f.fy[bj], f.fx[bi], acc[bj][bi]);
}

// What a workgroup needs to know about its part of a row, in one 512-byte record (two loads per lane, the
// first instructions of the kernel): the row's x blocks, the part's output blocks (at most 64) with their
// pair ranges, and for each of the eight waves the blocks it computes, as a 64-bit mask over the part's blocks.
// Blocks without pairs are in no mask.  With the pair ranges in the record the kernel reads no offsets table.
struct RowsRecord {
  int32_t row;                // -1: nothing to do
  int32_t x_first, x_count;   // the row's blocks in x
  int32_t o_first, o_count;   // the part's output blocks
  uint32_t empty_blocks[2];   // mask of the part's blocks that have no pair (they are written as zeros)
  int32_t pairs_end;          // end of the pair list of the part's last block
  uint32_t wave_blocks[kWaves][2];  // low and high word of wave w's mask
  int32_t downward;           // the waves take their blocks from the highest column down
  int32_t pad[39];
  int32_t pairs_begin[64];    // start of the pair list of block o_first + i (it ends where the next one starts)
};
static_assert(sizeof(RowsRecord) == BSA_ROWS_RECORD_INTS * 4, "record layout");

// cost of an output block in the list scheduling, in units of half a pair: its pairs and one write
constexpr int kBlockCost = 3;

// one wave per work table entry
__global__ __launch_bounds__(256) void rows_records_kernel(const int32_t *__restrict__ work_table, int64_t n_items,
                                                           int parts_log2, const int32_t *__restrict__ pair_offsets,
                                                           const int32_t *__restrict__ x_row_offsets,
                                                           const int32_t *__restrict__ o_row_offsets, int n_rows,
                                                           int64_t nnz_x, RowsRecord *__restrict__ records) {
  const int64_t at = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (at >= n_items) return;
  const int lane = threadIdx.x & 63;
  int32_t *out = reinterpret_cast<int32_t *>(records + at);
  int item = work_table ? work_table[at] : (int)at;
  item = __builtin_amdgcn_readfirstlane(item);
  const int downward = item >= 0 ? (item >> 30) & 1 : 0;
  if (item >= 0) item &= ~BSA_ROWS_DOWNWARD;
  const int part = item & ((1 << parts_log2) - 1);
  const int row = item < 0 ? -1 : item >> parts_log2;
  int value = 0, offset = 0;  // lane l writes ints l and 64 + l of the record
  if (row < 0 || row >= n_rows) {  // nothing, or a corrupt table (which must not turn into a wild read)
    if (lane == 0) value = -1;
  } else {
    int n0 = o_row_offsets[row], n1 = o_row_offsets[row + 1];
    if (parts_log2) {  // this part's run of the row's output blocks
      const int64_t len = n1 - n0;
      const int first = n0 + (int)((len * part) >> parts_log2), last = n0 + (int)((len * (part + 1)) >> parts_log2);
      n0 = first;
      n1 = last;
    }
    n0 = __builtin_amdgcn_readfirstlane(n0);
    n1 = __builtin_amdgcn_readfirstlane(n1);
    if (n1 - n0 > 64) n1 = n0;  // the caller sizes the parts; a part that does not fit a mask is refused whole
    const int xs = x_row_offsets[row];
    int nx = x_row_offsets[row + 1] - xs;
    if (xs < 0 || nx < 0 || (int64_t)xs + nx > nnz_x) nx = 0;
    // lane i: pair range of block n0 + i
    int my_pairs = 0;
    const int pairs_end = pair_offsets[n1];
    if (n0 + lane < n1) {
      offset = pair_offsets[n0 + lane];
      my_pairs = pair_offsets[n0 + lane + 1] - offset;
    }
    // blocks in ascending order, each to the wave with the least work so far (the lowest such wave)
    int load[kWaves];
    uint64_t blocks[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) load[w] = 0, blocks[w] = 0;
    for (int i = 0; i < n1 - n0; ++i) {
      const int c = __builtin_amdgcn_readlane(my_pairs, i);
      if (c <= 0) continue;
      int best = 0, least = load[0];
#pragma unroll
      for (int w = 1; w < kWaves; ++w)
        if (load[w] < least) best = w, least = load[w];
#pragma unroll
      for (int w = 0; w < kWaves; ++w)
        if (w == best) load[w] += 2 * c + kBlockCost, blocks[w] |= 1ull << i;
    }
    const uint64_t empty = __ballot(n0 + lane < n1 && my_pairs <= 0);
    if (lane == 0) value = n0 >= n1 ? -1 : row;
    else if (lane == 1) value = xs;
    else if (lane == 2) value = nx;
    else if (lane == 3) value = n0;
    else if (lane == 4) value = n1 - n0;
    else if (lane == 5) value = (int)(uint32_t)empty;
    else if (lane == 6) value = (int)(uint32_t)(empty >> 32);
    else if (lane == 7) value = pairs_end;
    else if (lane == 24) value = downward;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (lane == 8 + 2 * w) value = (int)(uint32_t)blocks[w];
      if (lane == 9 + 2 * w) value = (int)(uint32_t)(blocks[w] >> 32);
    }
  }
  out[lane] = value;
  out[64 + lane] = offset;
}

// One pair of a wave's walk; everything here is wave uniform (scalar registers).
struct PairItem {
  const char *y;  // the y block (for an item past the end: the last block requested, so the load hits)
  int xoff;       // offset of the x block in the panel, -1 if it is not resident
  int px;         // packed index of the x block (range checked), for the read from global memory
  int block;      // the output block the pair belongs to
  bool last;      // the block's last pair: the block is written after it
  bool valid;     // false: past the end of the wave's pairs
};

// One record: one part of a row.  `mine`: int `lane` of the record, `offs`: int 64 + lane (the pair list of
// the part's block `lane` starts there).  Every wave of the workgroup passes the
// same number of barriers (none when the record holds nothing, else two).
template <typename Tr>
__device__ __forceinline__ void rows_part(const char *__restrict__ x, const char *__restrict__ y,
                                          char *__restrict__ out, const int32_t *__restrict__ pair_offsets,
                                          const int32_t *__restrict__ pairs, const int mine, const int offs,
                                          int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, char *rows_smem,
                                          const int lane, const int wave) {
  const int row = __builtin_amdgcn_readlane(mine, 0);
  if (row < 0) return;
  const int xs = __builtin_amdgcn_readlane(mine, 1);
  int nx = __builtin_amdgcn_readlane(mine, 2);
  nx = nx < kPanelCap ? nx : kPanelCap;
  if (xs < 0 || xs + nx > nnz_x) nx = 0;
  char *panel = rows_smem;
  char *stage = rows_smem + kPanelCap * 8192 + wave * kStageBytes;

  // the row's x blocks into the panel: piece idx = 1 KiB = 8 rows; LDS slot (row, position) holds chunk
  // position ^ t_swizzle(row) of the row, so the lanes read the source permuted and land in lane order
  {
    const char *xsrc = x + (int64_t)xs * 8192;
    const int rl = lane >> 3;
    const int tsw = t_swizzle(rl);  // the swizzle of row 8 * piece + rl depends on rl only
    const uint32_t src_off = rl * 128 + (((lane & 7) ^ tsw) << 4);
    for (int idx = wave; idx < nx * 8; idx += kWaves) copy_1k_to_lds(xsrc + idx * 1024, src_off, panel + idx * 1024);
  }

  // the part's output blocks, and this wave's share of them (a corrupt record must not turn into a wild access)
  const int o_first = __builtin_amdgcn_readlane(mine, 3);
  int o_count = __builtin_amdgcn_readlane(mine, 4);
  if (o_first < 0 || o_count < 0 || o_count > 64 || (int64_t)o_first + o_count > nnz_o) o_count = 0;
  uint64_t todo = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(mine, 9 + 2 * wave) << 32) |
                  (uint32_t)__builtin_amdgcn_readlane(mine, 8 + 2 * wave);
  todo &= o_count >= 64 ? ~0ull : (1ull << o_count) - 1;

  // output blocks without pairs: zeros, block first + 8 m + wave by this wave
  {
    uint64_t zeros = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(mine, 6) << 32) |
                     (uint32_t)__builtin_amdgcn_readlane(mine, 5);
    zeros &= o_count >= 64 ? ~0ull : (1ull << o_count) - 1;
    zeros &= 0x0101010101010101ull << wave;
    while (zeros) {
      const int b = __builtin_ctzll(zeros);
      zeros &= zeros - 1;
      char *ob = out + (int64_t)(o_first + b) * 8192;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        __builtin_nontemporal_store(u32x4{0, 0, 0, 0}, reinterpret_cast<u32x4 *>(ob + i * 1024 + lane * 16));
    }
  }

  // The walk over this wave's pairs is scalar work without a branch: `todo` holds the wave's blocks from the
  // one being walked on (its lowest set bit, or its highest when the part is walked downward), [w_p, w_pe) are that block's pairs from the one handed out last.
  // step() moves to the next pair and requests its list entry; entry_to_item() turns the entry into addresses.
  // In the loop the two are called a whole pair of matrix products apart.  The entry is requested by a vector
  // load (every lane the same 8 bytes) from inline assembly and waited for with vmcnt like the y blocks: a
  // scalar load would share its counter with the LDS reads and, returning out of order, make every wait for an
  // LDS read a wait for the load as well.  Only the first three entries of a wave, in front of the loop, come
  // by scalar loads (behind the panel copies, a counted vector load would have to wait for those).
  const int pairs_end = __builtin_amdgcn_readlane(mine, 7);
  auto range_of = [&](int b, int &p, int &pe) {  // pair range of the part's block b (0 .. 63)
    p = __builtin_amdgcn_readlane(offs, b);
    const int next = __builtin_amdgcn_readlane(offs, (b + 1) & 63);
    pe = b + 1 < o_count ? next : pairs_end;
  };
  // A wave takes its blocks in ascending order of the column, or (downward) in descending order; the pairs of a
  // block are always walked in ascending order of k.
  const bool downward = __builtin_amdgcn_readlane(mine, 24) != 0;
  auto next_block = [&](uint64_t blocks) { return downward ? 63 - __builtin_clzll(blocks) : __builtin_ctzll(blocks); };
  int w_p = 0, w_pe = 0;
  if (todo) range_of(next_block(todo), w_p, w_pe);
  w_p -= 1;  // nothing handed out yet
  // what a step leaves for entry_to_item(): the entry (requested) and the facts known without it
  u32x2 raw_entry = {0, 0};
  int raw_block = 0;
  bool raw_last = false, raw_valid = false;
  uint32_t lane_zero = 0;
  asm volatile("" : "+v"(lane_zero));
  auto advance = [&]() -> const int32_t * {  // returns where the next pair's entry lies
    const int p1 = w_p + 1;
    const bool block_done = p1 >= w_pe && todo != 0;
    const uint64_t without = downward ? todo & ~(1ull << (63 - __builtin_clzll(todo | 1))) : todo & (todo - 1);
    const uint64_t rest = block_done ? without : todo;
    const int b = rest ? next_block(rest) : 0;
    int bp, bpe;
    range_of(b, bp, bpe);
    w_p = block_done ? bp : p1;
    w_pe = block_done ? bpe : w_pe;
    todo = rest;
    raw_valid = rest != 0;
    raw_block = o_first + b;
    raw_last = w_p + 1 >= w_pe;
    // past the end the last entry is requested again (the request must not depend on a branch)
    const int at = raw_valid ? w_p : (pairs_end > 0 ? pairs_end - 1 : 0);
    return pairs + 2 * (int64_t)(at < 0 ? 0 : at);
  };
  auto step_scalar = [&]() {
    const int32_t *src = advance();
    uint64_t e;  // spelled out: the compiler would pick a vector load, since the entry is kept in vector registers
    asm volatile("s_load_dwordx2 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e) : "s"(src) : "memory");
    raw_entry = u32x2{(uint32_t)e, (uint32_t)(e >> 32)};
  };
  auto step = [&]() {
    const int32_t *src = advance();
    asm volatile("s_nop 4\n\tglobal_load_dwordx2 %0, %1, %2" : "=v"(raw_entry) : "v"(lane_zero), "s"(src) : "memory");
  };
  const char *y_recent = y;
  auto entry_to_item = [&]() {
    PairItem it;
    it.valid = raw_valid;
    it.block = raw_block;
    it.last = raw_last;
    const int px = __builtin_amdgcn_readfirstlane((int)raw_entry[0]);
    const int py = __builtin_amdgcn_readfirstlane((int)raw_entry[1]);
    // a corrupt list must not turn into a wild read
    if (raw_valid) y_recent = y + (uint64_t)((py < 0 || py >= nnz_y) ? 0 : py) * 8192;
    it.y = y_recent;
    it.px = (px < 0 || px >= nnz_x) ? 0 : px;
    it.xoff = (unsigned)(px - xs) < (unsigned)nx ? (px - xs) * 8192 : -1;
    return it;
  };
  if (!todo) {
    // no block for this wave (none of its blocks has a pair: the list of pairs may be empty, so nothing is read
    // from it): its panel pieces and zero blocks must still land before the others read the panel
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    __syncthreads();
    return;
  }
  step_scalar();

  const uint32_t lane_lo = 16 * lane, lane_hi = 16 * lane + 4096;

  LaneAddr la;
  {
    const int li = lane & 31, kg = lane >> 5;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int rs = 8 * h + (lane >> 3);
      la.wr[h] = stage + rs * 128 + (((lane & 7) ^ y_swizzle(rs)) << 4);
    }
    const int g = lane >> 4, ls = lane & 15;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int rd = 0; rd < 2; ++rd) {
        const int rs = 8 * (g >> 1) + 4 * rd + (ls >> 2);
        const int col = 32 * b + 16 * (g & 1) + 4 * (ls & 3);
        la.tr[b][rd] = stage + rs * 128 + (((col >> 3) ^ y_swizzle(rs)) << 4) + ((col & 4) << 1);
      }
#pragma unroll
    for (int s = 0; s < 4; ++s) la.xoff[s] = li * 128 + (((2 * s + kg) ^ t_swizzle(li)) << 4);
  }

  f32x16 acc[2][2];  // [block along j][block along i]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // The registers of a slot are written by loads the compiler does not know of.  Two rules keep it from ever
  // touching them while a load is in flight: (1) no load sits in a branch of its own (a join could make the
  // compiler copy the registers), so blocks are requested unconditionally, the requests past the end of a wave's
  // pairs repeat its last block; (2) every request is consumed, the last ones by the statement after the loop
  // that passes both slots through (registers whose contents are never used may be reused at once).
  YSlot slot_a, slot_b;
  PairItem item_a = entry_to_item();
  step_scalar();
  PairItem item_b = entry_to_item();
  step_scalar();
  PairItem upcoming = entry_to_item();  // the pair after item_b
  y_issue(slot_a, item_a.y, lane_lo, lane_hi);
  y_issue(slot_b, item_b.y, lane_lo, lane_hi);
  // everything requested so far has arrived: the panel pieces of this wave and both slots
  BSA_Y_WAIT(slot_a, 0);
  BSA_Y_TIE(slot_b);
  __syncthreads();

  int flushed = 0;  // a block was written after the last pair

  // The loop is software pipelined across pairs: while the last two quarters of a pair are multiplied, the
  // first two quarters of the next pair are staged and their fragments read, so the matrix core does not wait
  // for LDS at the start of a pair.  f0 / f1 hold the fragments of the quarter multiplied next / after it.
  // Past the end of the wave's pairs the staging goes on with the block requested last (no branch; the
  // fragments are not used).
  Frags f0, f1;
  XSource x_cur;
  x_cur.resident = item_a.xoff >= 0;
  x_cur.lds = panel + (item_a.xoff >= 0 ? item_a.xoff : 0);
  x_cur.px = item_a.px;
  stage_and_read<0>(f0, slot_a, x_cur, la, x, lane);
  stage_and_read<1>(f1, slot_a, x_cur, la, x, lane);

  // the pair `cur` from `cur_slot` (its first two quarters are in f0 / f1 already); `next_slot` holds the pair
  // `next`; at the end `cur` is the pair whose block has been requested into `cur_slot`
  auto do_pair = [&](YSlot &cur_slot, PairItem &cur, YSlot &next_slot, const PairItem &next) {
    const PairItem fresh = upcoming;
    step();  // requests the list entry of the pair after `fresh`; it is read at the end of this pair
    XSource x_next;
    x_next.resident = next.xoff >= 0;
    x_next.lds = panel + (next.xoff >= 0 ? next.xoff : 0);
    x_next.px = next.px;
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f0);
    stage_and_read<2>(f0, cur_slot, x_cur, la, x, lane);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f1);
    stage_and_read<3>(f1, cur_slot, x_cur, la, x, lane);
    // the slot's registers have been handed to the LDS writes: request the block of the pair after next
    y_issue(cur_slot, fresh.y, lane_lo, lane_hi);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f0);
    // younger than the next slot's loads (issued during the pair before this one): the 8 loads just issued,
    // the request of the list entry at the top of this pair, and the 8 stores of a block written after that pair
    if (flushed)
      asm volatile("s_waitcnt vmcnt(17)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    BSA_Y_TIE(next_slot);
    flushed = 0;
    stage_and_read<0>(f0, next_slot, x_next, la, x, lane);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f1);
    stage_and_read<1>(f1, next_slot, x_next, la, x, lane);
    x_cur = x_next;
    // the list entry requested at the top of this pair: only the slot's 8 loads are younger.  One statement on
    // the straight path: the entry's registers pass through it, and with a wait in either branch of the test
    // below the compiler would merge two copies of them, made while the load may still be in flight.
    asm volatile("s_waitcnt vmcnt(8)" : "+v"(raw_entry) : : "memory");
    upcoming = entry_to_item();
    if (cur.last) {
      rows_flush<Tr>(acc, out + (int64_t)cur.block * 8192, stage, lane);
      flushed = 1;
    }
    cur = fresh;
  };
  while (true) {
    do_pair(slot_a, item_a, slot_b, item_b);
    if (!item_b.valid) break;
    do_pair(slot_b, item_b, slot_a, item_a);
    if (!item_a.valid) break;
  }
  // the last requests land here
  BSA_Y_WAIT(slot_a, 0);
  BSA_Y_TIE(slot_b);
  // the panel may be overwritten (by the next record's row) once every wave is done with it
  __syncthreads();
}

// Workgroup g runs on XCD g % 8 and takes the records 8 (items_per_wg (g / 8) + r) + g % 8, r = 0 ..
// items_per_wg - 1, one after the other: consecutive entries of its XCD's list in the work table.
template <typename Tr>
__global__ __launch_bounds__(kWaves * 64, 1) void matmul_rows_kernel(
    const char *__restrict__ x, const char *__restrict__ y, char *__restrict__ out,
    const int32_t *__restrict__ pair_offsets, const int32_t *__restrict__ pairs,
    const RowsRecord *__restrict__ records, int64_t n_items, int items_per_wg, int64_t nnz_o, int64_t nnz_x,
    int64_t nnz_y) {
  extern __shared__ __attribute__((aligned(16))) char rows_smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t group = blockIdx.x >> 3, xcd = blockIdx.x & 7;
  // lane l fetches ints l and 64 + l of a record; the next record is requested before the current one is worked on
  auto fetch = [&](int r, int &head, int &offs) {
    const int64_t at = 8 * (group * items_per_wg + r) + xcd;
    const bool there = at < n_items && r < items_per_wg;
    const int32_t *rec = reinterpret_cast<const int32_t *>(records + (there ? at : 0));
    head = rec[lane];
    offs = rec[64 + lane];
    if (!there) head = -1;  // int 0 of a record: -1 means nothing to do
  };
  int mine, offs;
  fetch(0, mine, offs);
  for (int r = 0; r < items_per_wg; ++r) {
    int mine_next, offs_next;
    fetch(r + 1, mine_next, offs_next);
    rows_part<Tr>(x, y, out, pair_offsets, pairs, mine, offs, nnz_o, nnz_x, nnz_y, rows_smem, lane, wave);
    mine = mine_next;
    offs = offs_next;
  }
}

template <typename Tr>
int launch_rows(const void *x, const void *y, void *out, const int32_t *pair_offsets, const int32_t *pairs,
                const int32_t *records, int64_t n_items, int items_per_wg, int64_t nnz_o, int64_t nnz_x,
                int64_t nnz_y, hipStream_t s) {
  static bool configured = false;  // raising the dynamic LDS limit is per function, once per process
  if (!configured) {
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&matmul_rows_kernel<Tr>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kRowsLds));
    configured = true;
  }
  // groups of 8 * items_per_wg records, one workgroup per XCD and group
  const int64_t groups = bsa::cdiv(n_items, (int64_t)8 * items_per_wg);
  matmul_rows_kernel<Tr><<<(unsigned)(groups * 8), kWaves * 64, kRowsLds, s>>>(
      static_cast<const char *>(x), static_cast<const char *>(y), static_cast<char *>(out), pair_offsets, pairs,
      reinterpret_cast<const RowsRecord *>(records), n_items, items_per_wg, nnz_o, nnz_x, nnz_y);
  return bsa::check_launch("matmul_rows_kernel");
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int bsa_matmul_rows_records(const int32_t *work_table, int64_t n_items, int parts_log2,
                                       const int32_t *pair_offsets, const int32_t *x_row_offsets,
                                       const int32_t *o_row_offsets, int64_t n_rows, int64_t n_cols,
                                       int64_t nnz_x, int32_t *records, bsa_stream_t stream) {
  const char *who = "bsa_matmul_rows_records";
  BSA_REQUIRE(parts_log2 >= 0 && parts_log2 <= 3, "%s: parts_log2 must be 0..3 (got %d)", who, parts_log2);
  BSA_REQUIRE(n_rows >= 0 && (n_rows << parts_log2) < (int64_t)BSA_ROWS_DOWNWARD, "%s: bad number of block rows", who);
  BSA_REQUIRE(n_items >= 0 && n_items < 0x7fffffffLL, "%s: bad number of table entries", who);
  BSA_REQUIRE(nnz_x >= 0, "%s: negative size", who);
  BSA_REQUIRE(n_cols >= 0 && ((n_cols + (1 << parts_log2) - 1) >> parts_log2) <= 64,
              "%s: a part of a row must hold at most 64 output blocks (%lld columns of blocks in %d parts)", who,
              (long long)n_cols, 1 << parts_log2);
  BSA_REQUIRE(work_table != nullptr || (parts_log2 == 0 && n_items == n_rows),
              "%s: without a work table the rows are taken whole and in order", who);
  if (n_items == 0) return BSA_OK;
  BSA_REQUIRE(pair_offsets && x_row_offsets && o_row_offsets && records, "%s: NULL pointer", who);
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(records) & 127) == 0, "%s: records must be 128-byte aligned", who);
  rows_records_kernel<<<(unsigned)bsa::cdiv(n_items, 4), 256, 0, bsa::as_stream(stream)>>>(
      work_table, n_items, parts_log2, pair_offsets, x_row_offsets, o_row_offsets, (int)n_rows, nnz_x,
      reinterpret_cast<RowsRecord *>(records));
  return bsa::check_launch("rows_records_kernel");
}

extern "C" int bsa_matmul_rows(const void *x, const void *y, void *out, const int32_t *pair_offsets,
                               const int32_t *pairs, const int32_t *records, int64_t n_items,
                               int items_per_workgroup, int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs,
                               int dtype, bsa_stream_t stream) {
  BSA_REQUIRE(sbs == 64, "bsa_matmul_rows: sbs must be 64 (got %d)", sbs);
  BSA_REQUIRE(dtype == BSA_F16 || dtype == BSA_BF16, "bsa_matmul_rows: dtype must be fp16 or bf16 (got %d)", dtype);
  BSA_REQUIRE(nnz_o >= 0 && nnz_x >= 0 && nnz_y >= 0, "bsa_matmul_rows: negative size");
  BSA_REQUIRE(n_items >= 0 && n_items < 0x7fffffffLL, "bsa_matmul_rows: bad number of records");
  BSA_REQUIRE(items_per_workgroup >= 1 && items_per_workgroup <= 64,
              "bsa_matmul_rows: items_per_workgroup must be 1..64 (got %d)", items_per_workgroup);
  if (nnz_o == 0 || n_items == 0) return BSA_OK;
  BSA_REQUIRE(out && pair_offsets && records, "bsa_matmul_rows: NULL pointer");
  BSA_REQUIRE(aligned16(x) && aligned16(y) && aligned16(out), "bsa_matmul_rows: buffers must be 16-byte aligned");
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(records) & 127) == 0, "bsa_matmul_rows: records must be 128-byte aligned");
  hipStream_t s = bsa::as_stream(stream);
  if (dtype == BSA_BF16) return launch_rows<MBf16>(x, y, out, pair_offsets, pairs, records, n_items, items_per_workgroup, nnz_o, nnz_x, nnz_y, s);
  return launch_rows<MF16>(x, y, out, pair_offsets, pairs, records, n_items, items_per_workgroup, nnz_o, nnz_x, nnz_y, s);
}
