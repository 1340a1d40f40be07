// Block-sparse flash attention forward on the fp32 matrix-core instruction (v_mfma_f32_16x16x4_f32): fp32
// operands of every block size, and 16-bit operands of the block sizes the 16-bit matrix-core kernel does not
// take (they are widened to fp32 while they are staged, probabilities are rounded to the operand type before
// they multiply V, as the reference does, blksprs/ops/flash_attention.py:1193).
//
// One workgroup owns one (batch entry, query block).  Its waves form G groups of sbs / 16 waves: the groups
// share the key list (group g takes the entries g, g + G, ...), each with its own LDS tile and its own running
// maximum, sum and output, which are merged through LDS at the end; within a group wave w owns the query rows
// 16 w .. 16 w + 15 and all head slices.  The split gives a query block G times as many waves in flight: one
// group alone spends its time waiting for the next K or V block (a few hundred matrix-core cycles of work per
// block against a memory latency several times that).
//
// The products are formed transposed (S^T = K Q^T, O^T = V^T P^T), so that a lane owns one query row
// (lane % 16) and, per 16 x 16 tile, four keys or four output columns (4 (lane / 16) + r): the softmax
// statistics are in-lane reductions plus two exchanges between the four lane groups, the accumulator layout of
// the score product is the operand layout of the value product (P never leaves registers), and the rescaling of
// O is a multiplication by a per-lane factor.
//
// The query block's head slices sit in LDS for the whole walk; K and V blocks pass through a group's LDS tile,
// one head slice at a time, widened to fp32.  Row stride of the tiles: sbs + 4 floats, which spreads the 16 rows of
// a 128-bit operand read over all banks and the four key rows of a 32-bit read over four bank groups.
//
// Score pipeline (log2 domain), in the reference's order (blksprs/ops/flash_attention.py:1058-1224): scale *
// q k^T, + bias, native causal predicate, explicit mask; inactive q / k head slices add nothing to the scores,
// inactive v slices nothing to the output; a row that sees nothing gives zeros and lse = -inf.
#include "attn_common.h"

namespace bsa {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename Tr>
struct Row4;  // four consecutive elements of a block row, widened

template <>
struct Row4<AttnF32> {
  __device__ static f32x4 load(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
  __device__ static void store(float *p, f32x4 v) { *reinterpret_cast<f32x4 *>(p) = v; }
};

template <typename Tr>
struct Row4 {
  typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
  __device__ static f32x4 load(const uint16_t *p) {
    const u16x4 h = *reinterpret_cast<const u16x4 *>(p);
    return f32x4{Tr::widen(h[0]), Tr::widen(h[1]), Tr::widen(h[2]), Tr::widen(h[3])};
  }
  __device__ static void store(uint16_t *p, f32x4 v) {
    *reinterpret_cast<u16x4 *>(p) = u16x4{Tr::round(v[0]), Tr::round(v[1]), Tr::round(v[2]), Tr::round(v[3])};
  }
};

// This lane's value and the value of lane ^ 16 (lane ^ 32), as (the one from the lower, the one from the upper
// group of 16 (32) lanes): v_permlane16_swap / v_permlane32_swap trade the odd groups of the first operand for the
// even groups of the second, so with the same value in both operands one result holds the even groups' values
// twice and the other the odd groups'.  One instruction, where a shuffle goes through LDS.
__device__ inline void pair16(float v, float &lower, float &upper) {
  // spelled out: both operands are read and written, and they must be two registers that hold the same value
  lower = upper = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
}
__device__ inline void pair32(float v, float &lower, float &upper) {
  lower = upper = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(lower), "+v"(upper));
}
// the larger of two values, NaN if either is
__device__ inline float nan_max(float a, float b) { return (b > a || b != b) ? b : a; }

template <int SBS>
struct F32mmaShape {
  static constexpr int kGroups = SBS == 64 ? 2 : 4;
  static constexpr int kStrips = SBS / 16;  // waves of a group
  static constexpr int kThreads = 64 * kStrips * kGroups;
  static constexpr int kLd = SBS + 4;
  // floats: one tile per group and the query block's head slices; or, at the end, every group's partial result
  static size_t lds_floats(int64_t nh, int nhv_max) {
    const size_t walk = (size_t)(kGroups + nh) * SBS * kLd;
    const size_t merge = (size_t)kGroups * SBS * (nhv_max * SBS + 2);
    return walk > merge ? walk : merge;
  }
};

template <typename Tr, int SBS, int NHV>
__global__ __launch_bounds__(F32mmaShape<SBS>::kThreads) void attn_fwd_f32mma_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  using Shape = F32mmaShape<SBS>;
  constexpr int kGroups = Shape::kGroups, kStrips = Shape::kStrips, kGroupThreads = 64 * kStrips;
  constexpr int kTiles = SBS / 16, kLd = Shape::kLd;
  extern __shared__ __attribute__((aligned(16))) float f32mma_smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int strip = wave % kStrips, group = wave / kStrips;
  const int in_group = threadIdx.x % kGroupThreads;
  float *tile = f32mma_smem + group * SBS * kLd;         // [SBS][kLd]: this group's K or V block
  float *qtile = f32mma_smem + kGroups * SBS * kLd;      // [nh][SBS][kLd]: the query block's head slices
  const int qrow = 16 * strip + (lane & 15), grp = lane >> 4;
  const int64_t b = blockIdx.x / a.nq, qb = blockIdx.x % a.nq;
  const int nh = (int)a.nh, nhv = (int)a.nhv;

  // the query block: inactive head slices stay out of the products (they add zeros to the scores)
  for (int h = group; h < nh; h += kGroups) {
    const int64_t pq = a.pidx_q[(b * a.nq + qb) * nh + h];
    if (pq >= 0 && pq < a.n_q_blocks) {
      const E *blk = static_cast<const E *>(a.q) + pq * SBS * SBS;
      for (int v = in_group; v < SBS * SBS / 4; v += kGroupThreads)
        *reinterpret_cast<f32x4 *>(qtile + h * SBS * kLd + ((4 * v) / SBS) * kLd + (4 * v) % SBS) =
            Row4<Tr>::load(blk + 4 * v);
    }
  }

  f32x4 oacc[NHV][kTiles];  // O^T: [value head slice][tile of 16 output columns], columns 4 grp + r of the tile
#pragma unroll
  for (int hv = 0; hv < NHV; ++hv)
#pragma unroll
    for (int c = 0; c < kTiles; ++c) oacc[hv][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  float row_m = -INFINITY, row_l = 0.f;  // running maximum of the row; this lane's share of the running sum

  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  const int64_t len = causal ? a.causal_lengths[b] : 0;
  const int k_begin = a.key_offsets[b * a.nq + qb], k_end = a.key_offsets[b * a.nq + qb + 1];
  // every group makes the same number of turns and passes the same barriers; a turn past the end of the list,
  // or a head slice that is not active, skips the work in between
  for (int e0 = k_begin; e0 < k_end; e0 += kGroups) {
    const int e = e0 + group;
    const bool turn = e < k_end;
    const int64_t kb = turn ? a.key_indices[e] : 0;
    // ---- S^T = K Q^T over the head slices: sacc[t][r] = score of (query qrow, key 16 t + 4 grp + r)
    f32x4 sacc[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) sacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int h = 0; h < nh; ++h) {
      const int64_t pq = a.pidx_q[(b * a.nq + qb) * nh + h];
      const int64_t pk = turn ? a.pidx_k[(b * a.nk + kb) * nh + h] : -1;
      const bool on = pq >= 0 && pk >= 0 && pq < a.n_q_blocks && pk < a.n_k_blocks;  // uniform over the group
      __syncthreads();  // the tile's readers are done
      if (on) {
        const E *blk = static_cast<const E *>(a.k) + pk * SBS * SBS;
        for (int v = in_group; v < SBS * SBS / 4; v += kGroupThreads)
          *reinterpret_cast<f32x4 *>(tile + ((4 * v) / SBS) * kLd + (4 * v) % SBS) = Row4<Tr>::load(blk + 4 * v);
      }
      __syncthreads();
      if (!on) continue;
      const float *qrow_p = qtile + h * SBS * kLd + qrow * kLd + 4 * grp;
#pragma unroll
      for (int s4 = 0; s4 < SBS / 16; ++s4) {
        // contraction steps 4 s4 .. 4 s4 + 3: lane group grp brings head dimensions 16 s4 + 4 grp + j
        const f32x4 qv = *reinterpret_cast<const f32x4 *>(qrow_p + 16 * s4);
#pragma unroll
        for (int t = 0; t < kTiles; ++t) {
          const f32x4 kv = *reinterpret_cast<const f32x4 *>(tile + (16 * t + (lane & 15)) * kLd + 16 * s4 + 4 * grp);
#pragma unroll
          for (int j = 0; j < 4; ++j) sacc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[j], qv[j], sacc[t], 0, 0, 0);
        }
      }
    }
    if (turn) {
      // ---- scale, bias, causal predicate, mask
      const int64_t pair = (b * a.nq + qb) * a.nk + kb;
      int64_t pb = -1, pm = -1;
      if (a.bias) {
        pb = a.pidx_bias[pair];
        if (pb >= a.n_bias_blocks) pb = -1;
      }
      if (a.mask) {
        pm = a.pidx_mask[pair];
        if (pm >= a.n_mask_blocks) pm = -1;
      }
      float tile_max = -INFINITY;
#pragma unroll
      for (int t = 0; t < kTiles; ++t) {
        const int key0 = 16 * t + 4 * grp;
        f32x4 s = sacc[t] * qk_scale;
        if (pb >= 0) s += Row4<Tr>::load(static_cast<const E *>(a.bias) + (pb * SBS + qrow) * SBS + key0) * kLog2e;
        uint32_t mbits = 0;
        if (pm >= 0) mbits = *reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(a.mask) +
                                                                  (pm * SBS + qrow) * SBS + key0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          bool off = ((mbits >> (8 * r)) & 0xffu) != 0;
          if (causal) {
            const int64_t qp = qb * SBS + qrow, kp = kb * SBS + key0 + r;
            off = off || kp > qp || qp >= len || kp >= len;
          }
          if (off) s[r] = -INFINITY;
          // a NaN score must not be dropped by the maximum: the row has to turn NaN as in the reference
          tile_max = (s[r] > tile_max || s[r] != s[r]) ? s[r] : tile_max;
        }
        sacc[t] = s;
      }
      // ---- online softmax of the row (its 4 lane groups hold different keys)
      {
        float lower, upper;
        pair16(tile_max, lower, upper);
        tile_max = nan_max(lower, upper);
        pair32(tile_max, lower, upper);
        tile_max = nan_max(lower, upper);
      }
      const float m_new = (tile_max > row_m || tile_max != tile_max) ? tile_max : row_m;
      const bool nothing = m_new == -INFINITY;  // the row has seen no key so far
      const float alpha = nothing ? 1.f : exp2f(row_m - m_new);
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = nothing ? 0.f : exp2f(sacc[t][r] - m_new);
          sum += p;
          sacc[t][r] = Tr::widen(Tr::round(p));
        }
      row_l = row_l * alpha + sum;
      row_m = m_new;
#pragma unroll
      for (int hv = 0; hv < NHV; ++hv)
#pragma unroll
        for (int c = 0; c < kTiles; ++c) oacc[hv][c] *= alpha;
    }
    // ---- O^T += V^T P^T, one value head slice at a time
#pragma unroll
    for (int hv = 0; hv < NHV; ++hv) {
      if (hv >= nhv) break;
      const int64_t pv = turn ? a.pidx_v[(b * a.nk + kb) * nhv + hv] : -1;
      const bool on = pv >= 0 && pv < a.n_v_blocks;  // uniform over the group
      __syncthreads();
      if (on) {
        const E *blk = static_cast<const E *>(a.v) + pv * SBS * SBS;
        for (int v = in_group; v < SBS * SBS / 4; v += kGroupThreads)
          *reinterpret_cast<f32x4 *>(tile + ((4 * v) / SBS) * kLd + (4 * v) % SBS) = Row4<Tr>::load(blk + 4 * v);
      }
      __syncthreads();
      if (!on) continue;
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float *vrow = tile + (16 * t + 4 * grp + r) * kLd + (lane & 15);
#pragma unroll
          for (int c = 0; c < kTiles; ++c)
            oacc[hv][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vrow[16 * c], sacc[t][r], oacc[hv][c], 0, 0, 0);
        }
    }
  }
  // ---- the row's sum over its four lane groups; then the groups' results are merged: every group leaves
  // (m, l, O) of its rows in LDS, group 0 rescales them to the common maximum and adds them up
  {
    float lower, upper;
    pair16(row_l, lower, upper);
    row_l = lower + upper;
    pair32(row_l, lower, upper);
    row_l = lower + upper;
  }
  constexpr int kRowFloats = NHV * SBS + 2;
  float *merge = f32mma_smem;  // [group][SBS][kRowFloats]
  __syncthreads();               // tiles and query slices are no longer read
  if (group != 0) {
    float *mine = merge + ((size_t)group * SBS + qrow) * kRowFloats;
    if (grp == 0) mine[0] = row_m, mine[1] = row_l;
#pragma unroll
    for (int hv = 0; hv < NHV; ++hv)
#pragma unroll
      for (int c = 0; c < kTiles; ++c) *reinterpret_cast<f32x4 *>(mine + 2 + hv * SBS + 16 * c + 4 * grp) = oacc[hv][c];
  }
  __syncthreads();
  if (group != 0) return;
#pragma unroll
  for (int g = 1; g < kGroups; ++g) {
    const float *other = merge + ((size_t)g * SBS + qrow) * kRowFloats;
    const float m_o = other[0], l_o = other[1];
    const float m_new = (m_o > row_m || m_o != m_o) ? m_o : row_m;
    const bool nothing = m_new == -INFINITY;
    const float mine_scale = nothing ? 1.f : exp2f(row_m - m_new), other_scale = nothing ? 1.f : exp2f(m_o - m_new);
    row_l = row_l * mine_scale + l_o * other_scale;
    row_m = m_new;
#pragma unroll
    for (int hv = 0; hv < NHV; ++hv)
#pragma unroll
      for (int c = 0; c < kTiles; ++c)
        oacc[hv][c] = oacc[hv][c] * mine_scale +
                      *reinterpret_cast<const f32x4 *>(other + 2 + hv * SBS + 16 * c + 4 * grp) * other_scale;
  }
  const float inv = row_l != 0.f ? 1.f / row_l : 0.f;
#pragma unroll
  for (int hv = 0; hv < NHV; ++hv) {
    if (hv >= nhv) break;
    const int64_t po = a.pidx_o[(b * a.nq + qb) * nhv + hv];
    if (po < 0 || po >= a.n_o_blocks) continue;
    E *orow = static_cast<E *>(a.o) + (po * SBS + qrow) * SBS + 4 * grp;
#pragma unroll
    for (int c = 0; c < kTiles; ++c) {
      f32x4 v = oacc[hv][c] * inv;
      if (row_l == 0.f) v = f32x4{0.f, 0.f, 0.f, 0.f};
      Row4<Tr>::store(orow + 16 * c, v);
    }
  }
  if (grp == 0) a.lse[(b * a.nq + qb) * SBS + qrow] = row_l != 0.f ? row_m + log2f(row_l) : -INFINITY;
}

template <typename Tr, int SBS, int NHV>
int launch_f32mma(const bsa_attn_args &a, hipStream_t s) {
  const size_t lds = F32mmaShape<SBS>::lds_floats(a.nh, NHV) * sizeof(float);
  static size_t configured = 0;  // the dynamic LDS limit of this instantiation, raised on demand
  if (lds > configured) {
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_fwd_f32mma_kernel<Tr, SBS, NHV>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    configured = lds;
  }
  attn_fwd_f32mma_kernel<Tr, SBS, NHV><<<(unsigned)(a.B * a.nq), F32mmaShape<SBS>::kThreads, lds, s>>>(a);
  return check_launch("attn_fwd_f32mma_kernel");
}

template <typename Tr, int SBS>
int launch_f32mma_slices(const bsa_attn_args &a, hipStream_t s) {
  if (a.nhv <= 1) return launch_f32mma<Tr, SBS, 1>(a, s);
  if (a.nhv == 2) return launch_f32mma<Tr, SBS, 2>(a, s);
  return launch_f32mma<Tr, SBS, 4>(a, s);
}

template <typename Tr>
int launch_f32mma_sizes(const bsa_attn_args &a, hipStream_t s) {
  if (a.sbs == 16) return launch_f32mma_slices<Tr, 16>(a, s);
  if (a.sbs == 32) return launch_f32mma_slices<Tr, 32>(a, s);
  return launch_f32mma_slices<Tr, 64>(a, s);
}

}  // namespace

// 1: not covered (more than four value head slices, or a query block whose head slices do not fit LDS)
int attn_fwd_f32mma(const bsa_attn_args &a, hipStream_t s) {
  if (a.B * a.nq == 0) return BSA_OK;
  if (a.nhv > 4) return 1;
  const int nhv_max = a.nhv <= 1 ? 1 : a.nhv == 2 ? 2 : 4;
  const size_t lds = (a.sbs == 16 ? F32mmaShape<16>::lds_floats(a.nh, nhv_max)
                      : a.sbs == 32 ? F32mmaShape<32>::lds_floats(a.nh, nhv_max)
                                    : F32mmaShape<64>::lds_floats(a.nh, nhv_max)) * sizeof(float);
  if (lds > 160 * 1024) return 1;
  if (a.dtype == BSA_F32) return launch_f32mma_sizes<AttnF32>(a, s);
  if (a.dtype == BSA_F16) return launch_f32mma_sizes<AttnF16>(a, s);
  return launch_f32mma_sizes<AttnBf16>(a, s);
}

}  // namespace bsa
