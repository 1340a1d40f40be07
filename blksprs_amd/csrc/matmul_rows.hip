// Row kernel of the block-sparse GEMM (16-bit operands, sbs == 64, untransposed operands): one workgroup of
// 8 waves owns one block row (b, i) of the output.
//
// x: the row's x blocks are consecutive in memory; up to 18 of them (144 KiB) are copied once into LDS by
// asynchronous global -> LDS copies and stay there while the waves walk the row's output blocks, so x is
// read from L2 once per row, and a wave never waits for x.  x blocks beyond the 18 resident ones are read
// from global memory in fragment layout (slow path, rare).
//
// Work split: the row's output blocks are cut into 8 contiguous runs of about equal numbers of (x, y) pairs
// (not of equal numbers of blocks), one run per wave; rows are handed to workgroups in the order the caller
// gives (longest first keeps the tail of the launch short).
//
// y: only y blocks stream.  A wave walks its slice of the pair list as one flat sequence.  Each y block
// travels global -> registers -> LDS -> matrix-core operand: two register slots of 8 KiB hold the y blocks of
// the next two pairs, so a block is requested about one and a half pairs before it is used.  The loads are
// issued from inline assembly and waited for with hand-placed s_waitcnt vmcnt(n): the compiler would join
// the outstanding loads with vmcnt(0) at every branch.  vmcnt counts vector memory instructions in issue
// order, so "all but the youngest n" is exact as long as n is not larger than the number of instructions
// issued after the loads waited for; every n used below is such a lower bound (the other slot's 8 loads,
// plus the 8 stores of an output block written since).
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
// 16 rows at a time and written with 16-byte stores that cover whole rows.
#include "attn_mfma_common.h"

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

// Rounds the tile, passes it through the wave's stage 16 rows at a time, writes it as one block with 16-byte
// stores that cover whole rows (8 stores per lane), and clears the accumulators.  A lane owns 4 columns of
// one of 32 rows per accumulator; v_permlane16_swap regroups the packed values so that, for each half of 16
// rows, all 64 lanes hold a piece (lanes 16 .. 31 and 48 .. 63 take over the right-hand column block of the
// rows of the lanes 16 below them).  Every lane takes part in every step: the exchange between lanes through
// LDS needs the wave to move as one.
template <typename Tr>
__device__ __forceinline__ void rows_flush(f32x16 (&acc)[2][2], char *ob, char *stage, int lane) {
  const int rr = lane & 15, quad = lane >> 4;
  // after the regrouping this lane holds row rr (or 16 + rr), column block quad % 2, column half quad / 2
  char *wbase = stage + rr * 128 + 8 * (quad >> 1);
  const int tw = t_swizzle(rr), cb = 4 * (quad & 1);
  u32x4 back[2][2][2];  // [row block][half of 16 rows][store]
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
    uint32_t lo[8], hi[8];  // [2 rq + word]: rows 0 .. 15 / rows 16 .. 31 of this row block
#pragma unroll
    for (int rq = 0; rq < 4; ++rq)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const uint32_t left = Tr::pack2(acc[0][bi][4 * rq + 2 * w], acc[0][bi][4 * rq + 2 * w + 1]);
        const uint32_t right = Tr::pack2(acc[1][bi][4 * rq + 2 * w], acc[1][bi][4 * rq + 2 * w + 1]);
        // lanes 16 .. 31 / 48 .. 63 of `left` trade places with lanes 0 .. 15 / 32 .. 47 of `right`
        const u32x2 sw = __builtin_bit_cast(u32x2, __builtin_amdgcn_permlane16_swap(left, right, false, false));
        lo[2 * rq + w] = sw[0];
        hi[2 * rq + w] = sw[1];
      }
    // LDS executes this wave's instructions in order: the reads of one step see its writes and are done
    // before the next step's writes land, so the four steps are queued without waiting in between (the wave
    // barriers only keep the compiler from reordering them; they emit nothing)
#pragma unroll
    for (int hr = 0; hr < 2; ++hr) {
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const u32x2 v = hr == 0 ? u32x2{lo[2 * rq], lo[2 * rq + 1]} : u32x2{hi[2 * rq], hi[2 * rq + 1]};
        // columns 32 (quad % 2) + 8 rq + 4 (quad / 2) .. + 3: chunk 4 (quad % 2) + rq
        *reinterpret_cast<u32x2 *>(wbase + (((cb + rq) ^ tw) << 4)) = v;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int q = t * 64 + lane;
        const int r = q >> 3, ch = q & 7;
        back[bi][hr][t] = *reinterpret_cast<const u32x4 *>(stage + r * 128 + ((ch ^ t_swizzle(r)) << 4));
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int hr = 0; hr < 2; ++hr)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int q = t * 64 + lane;
        const int r = q >> 3, ch = q & 7;
        // streaming store: the tile is not read again
        __builtin_nontemporal_store(
            back[bi][hr][t], reinterpret_cast<u32x4 *>(ob + (uint32_t)((32 * bi + 16 * hr + r) * 128 + ch * 16)));
      }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
}

// What a workgroup needs to know about its part of a row, in one 128-byte record (one load, where walking the
// tables is a chain of five dependent loads and a loop of ballots): the row, the x blocks of the row, and for
// each of the eight waves its run of output blocks and the pairs of that run.  Wave w takes the output blocks
// in front of which at least w / 8 and less than (w + 1) / 8 of the part's pairs lie.
struct RowsRecord {
  int32_t row;                    // -1: nothing to do
  int32_t x_first, x_count;       // the row's blocks in x
  int32_t pad0;
  int32_t block_begin[kWaves + 1];  // wave w: output blocks [block_begin[w], block_begin[w + 1])
  int32_t pair_begin[kWaves + 1];   // pair_offsets at those blocks
  int32_t pad1[32 - 4 - 2 * (kWaves + 1)];
};
static_assert(sizeof(RowsRecord) == BSA_ROWS_RECORD_INTS * 4, "record layout");

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
  const int part = item & ((1 << parts_log2) - 1);
  const int row = item < 0 ? -1 : item >> parts_log2;
  int value = 0;  // lane l writes int l of the record
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
    const int xs = x_row_offsets[row];
    int nx = x_row_offsets[row + 1] - xs;
    if (xs < 0 || nx < 0 || (int64_t)xs + nx > nnz_x) nx = 0;
    const int row_p0 = pair_offsets[n0], row_p1 = pair_offsets[n1];
    const int64_t span = row_p1 - row_p0;
    // lane w < 8 counts the blocks in front of wave w's boundary: pair_offsets ascends, one ballot per 64 blocks
    // for each boundary
    int below[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) below[w] = 0;
    for (int base = n0; base < n1; base += 64) {
      const int b = base + lane;
      const int off = b < n1 ? pair_offsets[b] : 0x7fffffff;
#pragma unroll
      for (int w = 1; w < kWaves; ++w) {
        const int lo = row_p0 + (int)((span * w + kWaves - 1) / kWaves);
        below[w] += __builtin_popcountll(__ballot(off < lo));
      }
    }
    int begin = n0;  // boundary number lane (for lanes 0 .. 8)
#pragma unroll
    for (int w = 1; w < kWaves; ++w)
      if (lane == w) begin = n0 + below[w];
    if (lane >= kWaves) begin = n1;
    const int pair_at = pair_offsets[begin];
    const int moved = __shfl(begin, lane - 4), moved_pair = __shfl(pair_at, lane - 4 - (kWaves + 1));
    if (lane == 0) value = n0 >= n1 ? -1 : row;
    else if (lane == 1) value = xs;
    else if (lane == 2) value = nx;
    else if (lane >= 4 && lane < 4 + kWaves + 1) value = moved;
    else if (lane >= 4 + kWaves + 1 && lane < 4 + 2 * (kWaves + 1)) value = moved_pair;
  }
  if (lane < BSA_ROWS_RECORD_INTS) out[lane] = value;
}

template <typename Tr>
__global__ __launch_bounds__(kWaves * 64, 1) void matmul_rows_kernel(
    const char *__restrict__ x, const char *__restrict__ y, char *__restrict__ out,
    const int32_t *__restrict__ pair_offsets, const int32_t *__restrict__ pairs,
    const RowsRecord *__restrict__ records, int64_t nnz_x, int64_t nnz_y) {
  extern __shared__ __attribute__((aligned(16))) char rows_smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // the grid has one workgroup per record; lane l < 32 fetches int l of it
  const int32_t *rec = reinterpret_cast<const int32_t *>(records + blockIdx.x);
  const int mine = rec[lane & 31];
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

  // this wave's run of output blocks and its pairs
  const int wb0 = __builtin_amdgcn_readlane(mine, 4 + wave), wb1 = __builtin_amdgcn_readlane(mine, 5 + wave);
  const int p_begin = __builtin_amdgcn_readlane(mine, 4 + kWaves + 1 + wave);
  const int p_end = __builtin_amdgcn_readlane(mine, 5 + kWaves + 1 + wave);

  // 64 entries of the pair list and 64 block boundaries at a time, one per lane.  A lane turns its entry into
  // what the loop needs per pair (the address of the y block; the panel offset of the x block, or -1 if it is
  // not resident), so that a pair costs a few v_readlane and no address arithmetic.
  int win_base = p_begin, win_px = 0, win_xoff = 0;
  uint32_t win_ylo = 0, win_yhi = 0;
  int off_base = wb0, win_off = 0;
  auto load_pair_window = [&](int base) {
    win_base = base;
    const int t = base + lane;
    int px = 0, py = 0;
    if (t < p_end) {
      const int2 v = *reinterpret_cast<const int2 *>(pairs + 2 * (int64_t)t);
      px = v.x;
      py = v.y;
    }
    // a corrupt list must not turn into a wild read
    const uint64_t ya = reinterpret_cast<uint64_t>(y) + (uint64_t)((py < 0 || py >= nnz_y) ? 0 : py) * 8192;
    win_ylo = (uint32_t)ya;
    win_yhi = (uint32_t)(ya >> 32);
    win_px = (px < 0 || px >= nnz_x) ? 0 : px;
    win_xoff = (unsigned)(px - xs) < (unsigned)nx ? (px - xs) * 8192 : -1;
    // a use right here: the wait for the load lands inside this (rarely taken) branch, not at the join
    asm volatile("" : "+v"(win_px), "+v"(win_xoff), "+v"(win_ylo), "+v"(win_yhi));
  };
  auto load_offset_window = [&](int base) {
    off_base = base;
    const int n = base + lane;
    win_off = pair_offsets[n <= wb1 ? n : wb1];
    asm volatile("" : "+v"(win_off));
  };
  // end of the pair list of block n (n < wb1)
  auto block_end = [&](int n) {
    if (n + 1 - off_base >= 64) load_offset_window(n);
    return __builtin_amdgcn_readlane(win_off, __builtin_amdgcn_readfirstlane(n + 1 - off_base));
  };
  // y block of pair t (clamped to the wave's last pair: the lookup stays in the window)
  auto y_block_of = [&](int t) -> const char * {
    t = t < p_end ? t : p_end - 1;
    const int sel = __builtin_amdgcn_readfirstlane(t - win_base);
    const uint32_t lo = __builtin_amdgcn_readlane(win_ylo, sel), hi = __builtin_amdgcn_readlane(win_yhi, sel);
    return reinterpret_cast<const char *>(((uint64_t)hi << 32) | lo);
  };
  load_pair_window(p_begin);
  load_offset_window(wb0);

  const uint32_t lane_lo = 16 * lane, lane_hi = 16 * lane + 4096;
  const bool has_pairs = p_begin < p_end;

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

  int cur = wb0;
  int blk_end = cur < wb1 ? block_end(cur) : -1;
  // writes the blocks that end at pair t (the first holds the sums, the others have no pairs: zeros)
  auto flush_until = [&](int t) {
    bool any = false;
    while (cur < wb1 && blk_end == t) {
      rows_flush<Tr>(acc, out + (int64_t)cur * 8192, stage, lane);
      any = true;
      ++cur;
      blk_end = cur < wb1 ? block_end(cur) : -1;
    }
    return any;
  };

  if (!has_pairs) {
    // only blocks without pairs (or none at all): wait for this wave's panel pieces, then write zeros
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    flush_until(p_begin);
    return;
  }

  // The registers of a slot are written by loads the compiler does not know of.  Two rules keep it from ever
  // touching them while a load is in flight: (1) no load sits in a branch of its own (a join could make the
  // compiler copy the registers), so blocks are requested unconditionally, the last two requests of a wave
  // repeat its last block; (2) every request is consumed, the last ones by the statement after the loop that
  // passes both slots through (registers whose contents are never used may be reused at once).
  YSlot slot_a, slot_b;
  y_issue(slot_a, y_block_of(p_begin), lane_lo, lane_hi);
  y_issue(slot_b, y_block_of(p_begin + 1), lane_lo, lane_hi);
  // everything requested so far has arrived: the panel pieces of this wave and both slots
  BSA_Y_WAIT(slot_a, 0);
  BSA_Y_TIE(slot_b);
  __syncthreads();

  int t = p_begin;
  int flushed = 0;  // a block was written after the last pair
  flush_until(t);   // blocks without pairs in front of the first pair

  // x block of pair t (the window must hold it)
  auto x_source_of = [&](int t) {
    const int sel = __builtin_amdgcn_readfirstlane(t - win_base);
    const int xoff = __builtin_amdgcn_readlane(win_xoff, sel);
    XSource src;
    src.resident = xoff >= 0;
    src.lds = panel + (xoff >= 0 ? xoff : 0);
    src.px = __builtin_amdgcn_readlane(win_px, sel);
    return src;
  };

  // The loop is software pipelined across pairs: while the last two quarters of pair t are multiplied, the
  // first two quarters of pair t + 1 are staged and their fragments read, so the matrix core does not wait
  // for LDS at the start of a pair.  f0 / f1 hold the fragments of the quarter multiplied next / after it.
  Frags f0, f1;
  XSource x_cur = x_source_of(t);
  stage_and_read<0>(f0, slot_a, x_cur, la, x, lane);
  stage_and_read<1>(f1, slot_a, x_cur, la, x, lane);

  // pair t from slot `cur_slot` (its first two quarters are in f0 / f1 already); `next_slot` holds pair t + 1
  auto do_pair = [&](YSlot &cur_slot, YSlot &next_slot) {
    // the window must hold pairs t .. t + 2
    if (t + 2 - win_base >= 64) load_pair_window(t);
    const char *next = y_block_of(t + 2);
    const bool more = t + 1 < p_end;
    const XSource x_next = x_source_of(more ? t + 1 : t);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f0);
    stage_and_read<2>(f0, cur_slot, x_cur, la, x, lane);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f1);
    stage_and_read<3>(f1, cur_slot, x_cur, la, x, lane);
    // the slot's registers have been handed to the LDS writes: request the block of the pair after next
    y_issue(cur_slot, next, lane_lo, lane_hi);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f0);
    // younger than the next slot's loads (issued during the pair before this one): the 8 loads just issued,
    // and the 8 stores of a block written after that pair
    if (flushed)
      asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    BSA_Y_TIE(next_slot);
    flushed = 0;
    if (more) stage_and_read<0>(f0, next_slot, x_next, la, x, lane);
    __builtin_amdgcn_sched_barrier(0);
    multiply<Tr>(acc, f1);
    if (more) stage_and_read<1>(f1, next_slot, x_next, la, x, lane);
    x_cur = x_next;
    ++t;
    if (flush_until(t)) flushed = 1;
  };
  while (t < p_end) {
    do_pair(slot_a, slot_b);
    if (t >= p_end) break;
    do_pair(slot_b, slot_a);
  }
  // the last requests land here
  BSA_Y_WAIT(slot_a, 0);
  BSA_Y_TIE(slot_b);
}

template <typename Tr>
int launch_rows(const void *x, const void *y, void *out, const int32_t *pair_offsets, const int32_t *pairs,
                const int32_t *records, int64_t n_items, int64_t nnz_x, int64_t nnz_y, hipStream_t s) {
  static bool configured = false;  // raising the dynamic LDS limit is per function, once per process
  if (!configured) {
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&matmul_rows_kernel<Tr>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kRowsLds));
    configured = true;
  }
  matmul_rows_kernel<Tr><<<(unsigned)n_items, kWaves * 64, kRowsLds, s>>>(
      static_cast<const char *>(x), static_cast<const char *>(y), static_cast<char *>(out), pair_offsets, pairs,
      reinterpret_cast<const RowsRecord *>(records), nnz_x, nnz_y);
  return bsa::check_launch("matmul_rows_kernel");
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

extern "C" int bsa_matmul_rows_records(const int32_t *work_table, int64_t n_items, int parts_log2,
                                       const int32_t *pair_offsets, const int32_t *x_row_offsets,
                                       const int32_t *o_row_offsets, int64_t n_rows, int64_t nnz_x,
                                       int32_t *records, bsa_stream_t stream) {
  const char *who = "bsa_matmul_rows_records";
  BSA_REQUIRE(parts_log2 >= 0 && parts_log2 <= 3, "%s: parts_log2 must be 0..3 (got %d)", who, parts_log2);
  BSA_REQUIRE(n_rows >= 0 && (n_rows << parts_log2) < 0x7fffffffLL, "%s: bad number of block rows", who);
  BSA_REQUIRE(n_items >= 0 && n_items < 0x7fffffffLL, "%s: bad number of table entries", who);
  BSA_REQUIRE(nnz_x >= 0, "%s: negative size", who);
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
                               const int32_t *pairs, const int32_t *records, int64_t n_items, int64_t nnz_o,
                               int64_t nnz_x, int64_t nnz_y, int sbs, int dtype, bsa_stream_t stream) {
  BSA_REQUIRE(sbs == 64, "bsa_matmul_rows: sbs must be 64 (got %d)", sbs);
  BSA_REQUIRE(dtype == BSA_F16 || dtype == BSA_BF16, "bsa_matmul_rows: dtype must be fp16 or bf16 (got %d)", dtype);
  BSA_REQUIRE(nnz_o >= 0 && nnz_x >= 0 && nnz_y >= 0, "bsa_matmul_rows: negative size");
  BSA_REQUIRE(n_items >= 0 && n_items < 0x7fffffffLL, "bsa_matmul_rows: bad number of records");
  if (nnz_o == 0 || n_items == 0) return BSA_OK;
  BSA_REQUIRE(out && pair_offsets && records, "bsa_matmul_rows: NULL pointer");
  BSA_REQUIRE(aligned16(x) && aligned16(y) && aligned16(out), "bsa_matmul_rows: buffers must be 16-byte aligned");
  BSA_REQUIRE((reinterpret_cast<uintptr_t>(records) & 127) == 0, "bsa_matmul_rows: records must be 128-byte aligned");
  hipStream_t s = bsa::as_stream(stream);
  if (dtype == BSA_BF16) return launch_rows<MBf16>(x, y, out, pair_offsets, pairs, records, n_items, nnz_x, nnz_y, s);
  return launch_rows<MF16>(x, y, out, pair_offsets, pairs, records, n_items, nnz_x, nnz_y, s);
}
