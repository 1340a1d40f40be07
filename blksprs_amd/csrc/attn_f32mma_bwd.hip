// Block-sparse flash attention backward on the fp32 matrix-core instruction (v_mfma_f32_16x16x4_f32), for the
// configurations attn_f32mma.hip computes forward: fp32 operands of every block size, 16-bit operands of the
// block sizes and head slice counts the 16-bit matrix-core kernels do not take (widened to fp32 while staged; P
// and dS are rounded to the operand type before they enter a product, as the reference does,
// blksprs/ops/flash_attention.py:1452, :1468, :1692).
//
// Three launches, no atomics, fixed summation order: delta = rowsum(o * dO); dK and dV of one (key block, head
// slice) per workgroup; dQ of one (query block, head slice) per workgroup.  A workgroup of the two main kernels
// keeps its own block's head slices (K and V, or Q and dO) in LDS for the whole walk and passes the other
// side's blocks through one LDS tile per group of waves.  Its waves form G groups that share the list of
// partner blocks (group g takes the entries g, g + G, ...) and add their partial gradients through LDS at the
// end; within a group wave w owns rows 16 w .. 16 w + 15 of the workgroup's own block.  Every product is formed
// so that a lane owns one row of the own block (lane % 16) and, per 16 x 16 tile, four rows of the partner block
// or four output columns (4 (lane / 16) + r): lse and delta are per-lane scalars in the dQ kernel, and P / dS
// pass from the accumulators of one product into the operands of the next without leaving registers.
//
// The scores are recomputed for every head slice (one workgroup per slice): every accumulator stays in registers,
// nothing is read-modify-written in global memory.  Score pipeline as in the forward kernel (log2 domain):
// scale * q k^T, + bias, native causal predicate, explicit mask; p = exp2(s - lse), 0 where lse = -inf.
#include "attn_common.h"

namespace bsa {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename Tr>
struct Quad;  // four consecutive elements of a block row, widened

template <>
struct Quad<AttnF32> {
  __device__ static f32x4 load(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
  __device__ static void store(float *p, f32x4 v) { *reinterpret_cast<f32x4 *>(p) = v; }
};

template <typename Tr>
struct Quad {
  typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
  __device__ static f32x4 load(const uint16_t *p) {
    const u16x4 h = *reinterpret_cast<const u16x4 *>(p);
    return f32x4{Tr::widen(h[0]), Tr::widen(h[1]), Tr::widen(h[2]), Tr::widen(h[3])};
  }
  __device__ static void store(uint16_t *p, f32x4 v) {
    *reinterpret_cast<u16x4 *>(p) = u16x4{Tr::round(v[0]), Tr::round(v[1]), Tr::round(v[2]), Tr::round(v[3])};
  }
};

template <int SBS>
struct BwdShape {
  static constexpr int kGroups = SBS == 64 ? 2 : 4;
  static constexpr int kStrips = SBS / 16;
  static constexpr int kGroupThreads = 64 * kStrips;
  static constexpr int kThreads = kGroupThreads * kGroups;
  static constexpr int kTiles = SBS / 16;
  static constexpr int kLd = SBS + 4;
  // floats: one tile per group and the own block's head slices; or, at the end, the groups' partial gradients
  static size_t lds_floats(int64_t own_slices) {
    const size_t walk = (size_t)(kGroups + own_slices) * SBS * kLd;
    const size_t merge = (size_t)kGroups * SBS * 2 * SBS;
    return walk > merge ? walk : merge;
  }
};

// the calling group's threads copy one sbs x sbs block into an LDS tile of fp32 rows of kLd floats
template <typename Tr, int SBS>
__device__ inline void stage(float *tile, const typename Tr::elem_t *blk, int in_group) {
  using S = BwdShape<SBS>;
  for (int v = in_group; v < SBS * SBS / 4; v += S::kGroupThreads)
    *reinterpret_cast<f32x4 *>(tile + ((4 * v) / SBS) * S::kLd + (4 * v) % SBS) = Quad<Tr>::load(blk + 4 * v);
}

// acc[t][r] += sum_d part[16 t + 4 grp + r][d] * own_row[d]: the rows of the partner tile against this lane's row
// of the own block (both with the contraction index along the row)
template <int SBS>
__device__ inline void mma_rows(f32x4 (&acc)[SBS / 16], const float *part, const float *own_row, int lane) {
  using S = BwdShape<SBS>;
  const int grp = lane >> 4;
#pragma unroll
  for (int s4 = 0; s4 < SBS / 16; ++s4) {
    const f32x4 bv = *reinterpret_cast<const f32x4 *>(own_row + 16 * s4 + 4 * grp);
#pragma unroll
    for (int t = 0; t < S::kTiles; ++t) {
      const f32x4 av = *reinterpret_cast<const f32x4 *>(part + (16 * t + (lane & 15)) * S::kLd + 16 * s4 + 4 * grp);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], bv[j], acc[t], 0, 0, 0);
    }
  }
}

// acc[c][r] += sum over the partner rows i = 16 t + 4 grp + r' of part[i][16 c + 4 grp_out + r] * w[t][r'], with
// w in the accumulator layout mma_rows leaves: the gradient of this lane's own row, columns 16 c + 4 grp + r
template <int SBS>
__device__ inline void mma_cols(f32x4 (&acc)[SBS / 16], const float *part, const f32x4 (&w)[SBS / 16], int lane) {
  using S = BwdShape<SBS>;
  const int grp = lane >> 4;
#pragma unroll
  for (int t = 0; t < S::kTiles; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float *row = part + (16 * t + 4 * grp + r) * S::kLd + (lane & 15);
#pragma unroll
      for (int c = 0; c < S::kTiles; ++c)
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(row[16 * c], w[t][r], acc[c], 0, 0, 0);
    }
}

// Turns raw products into scores of the log2 domain.  kOwnIsQuery: this lane's own row is the query (qi) and
// acc[t][r] belongs to key 16 t + 4 grp + r; otherwise the own row is the key (kj) and acc[t][r] belongs to query
// 16 t + 4 grp + r.
template <typename Tr, int SBS, bool kOwnIsQuery>
__device__ inline void to_scores(f32x4 (&acc)[SBS / 16], const bsa_attn_args &a, int64_t b, int64_t qb, int64_t kb,
                                 int own, int grp, float qk_scale, bool causal, int64_t len) {
  using E = typename Tr::elem_t;
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
#pragma unroll
  for (int t = 0; t < SBS / 16; ++t) {
    const int other0 = 16 * t + 4 * grp;
    f32x4 s = acc[t] * qk_scale;
    if (kOwnIsQuery) {
      if (pb >= 0) s += Quad<Tr>::load(static_cast<const E *>(a.bias) + (pb * SBS + own) * SBS + other0) * kLog2e;
      uint32_t mbits = 0;
      if (pm >= 0)
        mbits = *reinterpret_cast<const uint32_t *>(static_cast<const uint8_t *>(a.mask) + (pm * SBS + own) * SBS + other0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        bool off = ((mbits >> (8 * r)) & 0xffu) != 0;
        if (causal) {
          const int64_t qp = qb * SBS + own, kp = kb * SBS + other0 + r;
          off = off || kp > qp || qp >= len || kp >= len;
        }
        if (off) s[r] = -INFINITY;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int qi = other0 + r;
        if (pb >= 0) s[r] += Tr::widen(static_cast<const E *>(a.bias)[(pb * SBS + qi) * SBS + own]) * kLog2e;
        bool off = pm >= 0 && static_cast<const uint8_t *>(a.mask)[(pm * SBS + qi) * SBS + own] != 0;
        if (causal) {
          const int64_t qp = qb * SBS + qi, kp = kb * SBS + own;
          off = off || kp > qp || qp >= len || kp >= len;
        }
        if (off) s[r] = -INFINITY;
      }
    }
    acc[t] = s;
  }
}

// delta[b, qb, i] = sum over the active output slices of rowsum(o * dO); one wave per query block
template <typename Tr>
__global__ __launch_bounds__(64) void attn_f32mma_delta_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  const int sbs = a.sbs;
  const int64_t row = blockIdx.x;  // b * nq + qb
  const int lane = threadIdx.x;
  const int lanes_per_row = 64 / sbs > 0 ? 64 / sbs : 1;
  for (int i0 = 0; i0 < sbs; i0 += 64 / lanes_per_row) {
    const int i = i0 + lane / lanes_per_row;
    float acc = 0.f;
    if (i < sbs) {
      for (int64_t h = 0; h < a.nhv; ++h) {
        const int64_t po = a.pidx_o[row * a.nhv + h];
        if (po < 0 || po >= a.n_o_blocks) continue;
        const E *ob = static_cast<const E *>(a.o) + po * sbs * sbs + i * sbs;
        const E *gb = static_cast<const E *>(a.d_o) + po * sbs * sbs + i * sbs;
        for (int c = lane % lanes_per_row; c < sbs; c += lanes_per_row) acc = fmaf(Tr::widen(ob[c]), Tr::widen(gb[c]), acc);
      }
    }
    for (int d = 1; d < lanes_per_row; d <<= 1) acc += __shfl_xor(acc, d);
    if (i < sbs && (lane % lanes_per_row) == 0) a.delta[row * sbs + i] = acc;
  }
}

// adds the groups' partial gradients (two accumulators of SBS columns per own row) and leaves the sum in group 0
template <int SBS>
__device__ inline void merge_groups(f32x4 (&g0)[SBS / 16], f32x4 (&g1)[SBS / 16], float *smem, int group, int own,
                                    int grp) {
  using S = BwdShape<SBS>;
  __syncthreads();  // tiles and resident slices are no longer read
  float *mine = smem + ((size_t)group * SBS + own) * 2 * SBS;
  if (group != 0) {
#pragma unroll
    for (int c = 0; c < S::kTiles; ++c) {
      *reinterpret_cast<f32x4 *>(mine + 16 * c + 4 * grp) = g0[c];
      *reinterpret_cast<f32x4 *>(mine + SBS + 16 * c + 4 * grp) = g1[c];
    }
  }
  __syncthreads();
  if (group != 0) return;
#pragma unroll
  for (int g = 1; g < S::kGroups; ++g) {
    const float *other = smem + ((size_t)g * SBS + own) * 2 * SBS;
#pragma unroll
    for (int c = 0; c < S::kTiles; ++c) {
      g0[c] += *reinterpret_cast<const f32x4 *>(other + 16 * c + 4 * grp);
      g1[c] += *reinterpret_cast<const f32x4 *>(other + SBS + 16 * c + 4 * grp);
    }
  }
}

// grid (B * nk, max(nh, nhv)): dK slice h and dV slice h of one key block, dBias by slice 0
template <typename Tr, int SBS>
__global__ __launch_bounds__(BwdShape<SBS>::kThreads) void attn_f32mma_dkdv_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  using S = BwdShape<SBS>;
  constexpr int kTiles = S::kTiles, kLd = S::kLd;
  extern __shared__ __attribute__((aligned(16))) float f32mma_bwd_smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int strip = wave % S::kStrips, group = wave / S::kStrips, in_group = threadIdx.x % S::kGroupThreads;
  const int kj = 16 * strip + (lane & 15), grp = lane >> 4;  // this lane's key row
  const int64_t b = blockIdx.x / a.nk, kb = blockIdx.x % a.nk;
  const int64_t h = blockIdx.y;
  const int nh = (int)a.nh, nhv = (int)a.nhv;
  float *tile = f32mma_bwd_smem + group * SBS * kLd;
  float *ktile = f32mma_bwd_smem + S::kGroups * SBS * kLd;  // [nh][SBS][kLd]
  float *vtile = ktile + (size_t)nh * SBS * kLd;            // [nhv][SBS][kLd]
  int64_t pk = -1, pv = -1;
  if (h < nh) pk = a.pidx_k[(b * a.nk + kb) * nh + h];
  if (h < nhv) pv = a.pidx_v[(b * a.nk + kb) * nhv + h];
  if (pk >= a.n_k_blocks) pk = -1;
  if (pv >= a.n_v_blocks) pv = -1;
  const bool want_dbias = h == 0 && a.dbias != nullptr;
  if (pk < 0 && pv < 0 && !want_dbias) return;

  for (int s = group; s < nh + nhv; s += S::kGroups) {
    const bool is_k = s < nh;
    const int64_t p = is_k ? a.pidx_k[(b * a.nk + kb) * nh + s] : a.pidx_v[(b * a.nk + kb) * nhv + (s - nh)];
    if (p < 0 || p >= (is_k ? a.n_k_blocks : a.n_v_blocks)) continue;
    stage<Tr, SBS>(ktile + (size_t)s * SBS * kLd, static_cast<const E *>(is_k ? a.k : a.v) + p * SBS * SBS, in_group);
  }

  f32x4 dk[kTiles], dv[kTiles];
#pragma unroll
  for (int c = 0; c < kTiles; ++c) dk[c] = dv[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  const int64_t len = causal ? a.causal_lengths[b] : 0;
  const int q_begin = a.query_offsets[b * a.nk + kb], q_end = a.query_offsets[b * a.nk + kb + 1];
  for (int e0 = q_begin; e0 < q_end; e0 += S::kGroups) {
    const int e = e0 + group;
    const bool turn = e < q_end;
    const int64_t qb = turn ? a.query_indices[e] : 0;
    // ---- S[query][key] = Q K^T over the head slices; acc[t][r]: query 16 t + 4 grp + r against key kj
    f32x4 sacc[kTiles], dp[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) sacc[t] = dp[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nh; ++s) {
      const int64_t pq = turn ? a.pidx_q[(b * a.nq + qb) * nh + s] : -1;
      const int64_t pks = a.pidx_k[(b * a.nk + kb) * nh + s];
      const bool on = pq >= 0 && pks >= 0 && pq < a.n_q_blocks && pks < a.n_k_blocks;
      __syncthreads();
      if (on) stage<Tr, SBS>(tile, static_cast<const E *>(a.q) + pq * SBS * SBS, in_group);
      __syncthreads();
      if (on) mma_rows<SBS>(sacc, tile, ktile + (size_t)s * SBS * kLd + kj * kLd, lane);
    }
    if (turn) {
      to_scores<Tr, SBS, false>(sacc, a, b, qb, kb, kj, grp, qk_scale, causal, len);
      const float *lse = a.lse + (b * a.nq + qb) * SBS;
#pragma unroll
      for (int t = 0; t < kTiles; ++t) {
        const f32x4 l4 = *reinterpret_cast<const f32x4 *>(lse + 16 * t + 4 * grp);
#pragma unroll
        for (int r = 0; r < 4; ++r) sacc[t][r] = l4[r] != -INFINITY ? exp2f(sacc[t][r] - l4[r]) : 0.f;
      }
    }
    // ---- dP = dO V^T over the value slices, and dV_h += round(P)^T dO_h while dO_h is in the tile
    f32x4 prnd[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) prnd[t][r] = Tr::widen(Tr::round(sacc[t][r]));
    for (int s = 0; s < nhv; ++s) {
      const int64_t po = turn ? a.pidx_o[(b * a.nq + qb) * nhv + s] : -1;
      const int64_t pvs = a.pidx_v[(b * a.nk + kb) * nhv + s];
      const bool has_o = po >= 0 && po < a.n_o_blocks;
      const bool both = has_o && pvs >= 0 && pvs < a.n_v_blocks;
      const bool for_dv = has_o && s == h && pv >= 0;
      __syncthreads();
      if (both || for_dv) stage<Tr, SBS>(tile, static_cast<const E *>(a.d_o) + po * SBS * SBS, in_group);
      __syncthreads();
      if (both) mma_rows<SBS>(dp, tile, vtile + (size_t)s * SBS * kLd + kj * kLd, lane);
      if (for_dv) mma_cols<SBS>(dv, tile, prnd, lane);
    }
    // ---- dS = P (dP - delta); dBias; dK_h += scale * round(dS)^T Q_h
    if (turn) {
      const float *delta = a.delta + (b * a.nq + qb) * SBS;
      int64_t pb = -1;
      if (want_dbias) {
        pb = a.pidx_bias[(b * a.nq + qb) * a.nk + kb];
        if (pb >= a.n_bias_blocks) pb = -1;
      }
#pragma unroll
      for (int t = 0; t < kTiles; ++t) {
        const f32x4 d4 = *reinterpret_cast<const f32x4 *>(delta + 16 * t + 4 * grp);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float ds = sacc[t][r] * (dp[t][r] - d4[r]);
          // every (query block, key block) pair is visited once, so this is a plain store
          if (pb >= 0) a.dbias[(pb * SBS + 16 * t + 4 * grp + r) * SBS + kj] = ds;
          sacc[t][r] = Tr::widen(Tr::round(ds));
        }
      }
    }
    {
      const int64_t pq = turn && pk >= 0 ? a.pidx_q[(b * a.nq + qb) * nh + h] : -1;
      const bool on = pq >= 0 && pq < a.n_q_blocks;
      __syncthreads();
      if (on) stage<Tr, SBS>(tile, static_cast<const E *>(a.q) + pq * SBS * SBS, in_group);
      __syncthreads();
      if (on) mma_cols<SBS>(dk, tile, sacc, lane);
    }
  }
  merge_groups<SBS>(dk, dv, f32mma_bwd_smem, group, kj, grp);
  if (group != 0) return;
#pragma unroll
  for (int c = 0; c < kTiles; ++c) {
    if (pk >= 0) Quad<Tr>::store(static_cast<E *>(a.dk) + (pk * SBS + kj) * SBS + 16 * c + 4 * grp, dk[c] * a.scale);
    if (pv >= 0) Quad<Tr>::store(static_cast<E *>(a.dv) + (pv * SBS + kj) * SBS + 16 * c + 4 * grp, dv[c]);
  }
}

// grid (B * nq, nh): dQ slice h of one query block
template <typename Tr, int SBS>
__global__ __launch_bounds__(BwdShape<SBS>::kThreads) void attn_f32mma_dq_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  using S = BwdShape<SBS>;
  constexpr int kTiles = S::kTiles, kLd = S::kLd;
  extern __shared__ __attribute__((aligned(16))) float f32mma_bwd_smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int strip = wave % S::kStrips, group = wave / S::kStrips, in_group = threadIdx.x % S::kGroupThreads;
  const int qi = 16 * strip + (lane & 15), grp = lane >> 4;  // this lane's query row
  const int64_t b = blockIdx.x / a.nq, qb = blockIdx.x % a.nq;
  const int64_t h = blockIdx.y;
  const int nh = (int)a.nh, nhv = (int)a.nhv;
  float *tile = f32mma_bwd_smem + group * SBS * kLd;
  float *qtile = f32mma_bwd_smem + S::kGroups * SBS * kLd;  // [nh][SBS][kLd]
  float *gtile = qtile + (size_t)nh * SBS * kLd;            // [nhv][SBS][kLd]: dO
  const int64_t pq = a.pidx_q[(b * a.nq + qb) * nh + h];
  if (pq < 0 || pq >= a.n_q_blocks) return;

  for (int s = group; s < nh + nhv; s += S::kGroups) {
    const bool is_q = s < nh;
    const int64_t p = is_q ? a.pidx_q[(b * a.nq + qb) * nh + s] : a.pidx_o[(b * a.nq + qb) * nhv + (s - nh)];
    if (p < 0 || p >= (is_q ? a.n_q_blocks : a.n_o_blocks)) continue;
    stage<Tr, SBS>(qtile + (size_t)s * SBS * kLd, static_cast<const E *>(is_q ? a.q : a.d_o) + p * SBS * SBS, in_group);
  }

  f32x4 dq[kTiles], unused[kTiles];
#pragma unroll
  for (int c = 0; c < kTiles; ++c) dq[c] = unused[c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  const int64_t len = causal ? a.causal_lengths[b] : 0;
  const float lse = a.lse[(b * a.nq + qb) * SBS + qi], delta = a.delta[(b * a.nq + qb) * SBS + qi];
  const int k_begin = a.key_offsets[b * a.nq + qb], k_end = a.key_offsets[b * a.nq + qb + 1];
  for (int e0 = k_begin; e0 < k_end; e0 += S::kGroups) {
    const int e = e0 + group;
    const bool turn = e < k_end;
    const int64_t kb = turn ? a.key_indices[e] : 0;
    // ---- S^T[key][query] = K Q^T and dP^T = V dO^T; acc[t][r]: key 16 t + 4 grp + r against query qi
    f32x4 sacc[kTiles], dp[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) sacc[t] = dp[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nh; ++s) {
      const int64_t pqs = a.pidx_q[(b * a.nq + qb) * nh + s];
      const int64_t pks = turn ? a.pidx_k[(b * a.nk + kb) * nh + s] : -1;
      const bool on = pqs >= 0 && pks >= 0 && pqs < a.n_q_blocks && pks < a.n_k_blocks;
      __syncthreads();
      if (on) stage<Tr, SBS>(tile, static_cast<const E *>(a.k) + pks * SBS * SBS, in_group);
      __syncthreads();
      if (on) mma_rows<SBS>(sacc, tile, qtile + (size_t)s * SBS * kLd + qi * kLd, lane);
    }
    for (int s = 0; s < nhv; ++s) {
      const int64_t po = a.pidx_o[(b * a.nq + qb) * nhv + s];
      const int64_t pvs = turn ? a.pidx_v[(b * a.nk + kb) * nhv + s] : -1;
      const bool on = po >= 0 && pvs >= 0 && po < a.n_o_blocks && pvs < a.n_v_blocks;
      __syncthreads();
      if (on) stage<Tr, SBS>(tile, static_cast<const E *>(a.v) + pvs * SBS * SBS, in_group);
      __syncthreads();
      if (on) mma_rows<SBS>(dp, tile, gtile + (size_t)s * SBS * kLd + qi * kLd, lane);
    }
    if (turn) {
      to_scores<Tr, SBS, true>(sacc, a, b, qb, kb, qi, grp, qk_scale, causal, len);
#pragma unroll
      for (int t = 0; t < kTiles; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = lse != -INFINITY ? exp2f(sacc[t][r] - lse) : 0.f;
          sacc[t][r] = Tr::widen(Tr::round(p * (dp[t][r] - delta)));
        }
    }
    // ---- dQ_h += scale * round(dS) K_h
    {
      const int64_t pks = turn ? a.pidx_k[(b * a.nk + kb) * nh + h] : -1;
      const bool on = pks >= 0 && pks < a.n_k_blocks;
      __syncthreads();
      if (on) stage<Tr, SBS>(tile, static_cast<const E *>(a.k) + pks * SBS * SBS, in_group);
      __syncthreads();
      if (on) mma_cols<SBS>(dq, tile, sacc, lane);
    }
  }
  merge_groups<SBS>(dq, unused, f32mma_bwd_smem, group, qi, grp);
  if (group != 0) return;
#pragma unroll
  for (int c = 0; c < kTiles; ++c)
    Quad<Tr>::store(static_cast<E *>(a.dq) + (pq * SBS + qi) * SBS + 16 * c + 4 * grp, dq[c] * a.scale);
}

// dq, dk, dv (and the bias gradient) set to zero by ONE launch: the lengths one after the other
template <typename E>
__global__ void f32mma_zero_kernel(E *dq, int64_t n_dq, E *dk, int64_t n_dk, E *dv, int64_t n_dv, float *dbias,
                                   int64_t n_dbias) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t total = n_dq + n_dk + n_dv + n_dbias;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    if (i < n_dq) dq[i] = (E)0;
    else if (i < n_dq + n_dk) dk[i - n_dq] = (E)0;
    else if (i < n_dq + n_dk + n_dv) dv[i - n_dq - n_dk] = (E)0;
    else dbias[i - n_dq - n_dk - n_dv] = 0.f;
  }
}

template <typename E>
int zero_fill(E *dq, int64_t n_dq, E *dk, int64_t n_dk, E *dv, int64_t n_dv, float *dbias, int64_t n_dbias,
              hipStream_t s) {
  n_dq = dq && n_dq > 0 ? n_dq : 0;
  n_dk = dk && n_dk > 0 ? n_dk : 0;
  n_dv = dv && n_dv > 0 ? n_dv : 0;
  n_dbias = dbias && n_dbias > 0 ? n_dbias : 0;
  const int64_t total = n_dq + n_dk + n_dv + n_dbias;
  if (total == 0) return BSA_OK;
  int64_t blocks = cdiv(total, (int64_t)256);
  if (blocks > 65536) blocks = 65536;
  f32mma_zero_kernel<E><<<(unsigned)blocks, 256, 0, s>>>(dq, n_dq, dk, n_dk, dv, n_dv, dbias, n_dbias);
  return check_launch("f32mma_zero_kernel");
}

template <typename Tr, int SBS>
int bwd_f32mma(const bsa_attn_args &a, hipStream_t s) {
  using E = typename Tr::elem_t;
  using S = BwdShape<SBS>;
  const int64_t bs = (int64_t)SBS * SBS;
  // blocks no workgroup reaches (inactive counterpart slices) and bias blocks outside the attention layout stay zero
  if (int rc = zero_fill(static_cast<E *>(a.dq), a.n_q_blocks * bs, static_cast<E *>(a.dk), a.n_k_blocks * bs,
                         static_cast<E *>(a.dv), a.n_v_blocks * bs, a.dbias, a.n_bias_blocks * bs, s))
    return rc;
  const int64_t qrows = a.B * a.nq, krows = a.B * a.nk;
  if (qrows > 0) {
    attn_f32mma_delta_kernel<Tr><<<(unsigned)qrows, 64, 0, s>>>(a);
    if (int rc = check_launch("attn_f32mma_delta_kernel")) return rc;
  }
  const size_t lds = S::lds_floats(a.nh + a.nhv) * sizeof(float);
  static size_t configured = 0;  // the dynamic LDS limit of these instantiations, raised on demand
  if (lds > configured) {
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_f32mma_dkdv_kernel<Tr, SBS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    BSA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_f32mma_dq_kernel<Tr, SBS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    configured = lds;
  }
  const int64_t slices = a.nh > a.nhv ? a.nh : a.nhv;
  if (krows > 0 && (slices > 0 || a.dbias)) {
    dim3 grid((unsigned)krows, (unsigned)(slices > 0 ? slices : 1));
    attn_f32mma_dkdv_kernel<Tr, SBS><<<grid, S::kThreads, lds, s>>>(a);
    if (int rc = check_launch("attn_f32mma_dkdv_kernel")) return rc;
  }
  if (qrows > 0 && a.nh > 0) {
    dim3 grid((unsigned)qrows, (unsigned)a.nh);
    attn_f32mma_dq_kernel<Tr, SBS><<<grid, S::kThreads, lds, s>>>(a);
    if (int rc = check_launch("attn_f32mma_dq_kernel")) return rc;
  }
  return BSA_OK;
}

template <typename Tr>
int bwd_f32mma_sizes(const bsa_attn_args &a, hipStream_t s) {
  if (a.sbs == 16) return bwd_f32mma<Tr, 16>(a, s);
  if (a.sbs == 32) return bwd_f32mma<Tr, 32>(a, s);
  return bwd_f32mma<Tr, 64>(a, s);
}

}  // namespace

// 1: not covered (the head slices of a block do not fit LDS)
int attn_bwd_f32mma(const bsa_attn_args &a, hipStream_t s) {
  const size_t lds = (a.sbs == 16 ? BwdShape<16>::lds_floats(a.nh + a.nhv)
                      : a.sbs == 32 ? BwdShape<32>::lds_floats(a.nh + a.nhv)
                                    : BwdShape<64>::lds_floats(a.nh + a.nhv)) * sizeof(float);
  if (lds > 160 * 1024) return 1;
  if (a.dtype == BSA_F32) return bwd_f32mma_sizes<AttnF32>(a, s);
  if (a.dtype == BSA_F16) return bwd_f32mma_sizes<AttnF16>(a, s);
  return bwd_f32mma_sizes<AttnBf16>(a, s);
}

}  // namespace bsa
