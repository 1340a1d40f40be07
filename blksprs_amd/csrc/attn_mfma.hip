// Block-sparse flash attention on the matrix cores: fp16 / bf16 operands, sbs == 64,
// one or two 64-wide head slices for q/k and for v/o.
//
// Forward.  One workgroup of two waves owns one 64-row query block of one batch
// entry; each wave owns 32 query rows and walks the active key blocks of the row.
// The products are formed transposed, so that a lane owns ONE query row:
//
//   S^T[j][i] = sum_d K[j][d] Q[i][d]      A = K fragment (from LDS), B = Q fragment (registers)
//   O^T[d][i] = sum_j V[j][d] P^T[j][i]    A = V fragment (from LDS), B = P^T (registers)
//
// In the 32x32 accumulator layout lane l holds column i = l % 32 and, in register r,
// row 8 (r / 4) + 4 (l / 32) + r % 4.  The softmax statistics of a query row are
// therefore 16-register reductions inside a lane plus one exchange with lane l ^ 32,
// and the probabilities of S^T are, as they sit in registers, the B operand of the
// second product: registers 8u .. 8u+7 of key half jb cover keys
// 32 jb + 16 u + {4 kg .. 4 kg + 3, 8 + 4 kg .. 8 + 4 kg + 3} (kg = l / 32), and the V
// fragment is gathered from LDS for exactly that key set.  V is kept in LDS as
// (j, j+1) pairs per column (interleaved in registers with v_perm_b32 before the LDS
// write) so that its fragment is four conflict-free 32-bit reads; K is kept row-major
// with XOR-swizzled 16-byte chunks and its fragment is one 128-bit read.
//
// The K / V tiles of key block e+1, the mask words of e+1, the packed indices of e+2
// and the key index of e+3 are all fetched while block e is computed.  The index
// fetches use vector loads on purpose: they complete in order with the tile loads, so
// the one wait at the top of an iteration covers them and no scalar-load wait lands
// in front of an LDS read.
//
// Score pipeline (log2 domain), in this order: scale * q k^T, + bias, native causal
// predicate, explicit mask; probabilities are rounded to the operand type before they
// multiply V; the row sum uses the unrounded values.
#include "attn_common.h"

namespace bsa {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct MBf16 {
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static float widen(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }
};

struct MF16 {
  __device__ static f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
  }
  __device__ static uint32_t pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  __device__ static float widen(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
};

constexpr int kSbs = 64;
constexpr int kBlockBytes = kSbs * kSbs * 2;  // one 16-bit block
constexpr int kFwdThreads = 128;

// dword offset of column c in a pair row of the (j, j+1)-packed V tile; the placement of the column
// quads keeps both the 128-bit writes of the staging step and the 32-bit fragment reads conflict free
__device__ inline int pair_col_offset(int c) {
  const int q = c >> 2, a = q >> 1, h = q & 1;
  const int pos = ((a + 4 * h) & 7) + 8 * h;
  return 4 * pos + (c & 3);
}

// keeps a wave-uniform value in a vector register so that loads addressed with it use the vector memory path
__device__ inline int as_vector(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

__device__ inline int first_lane(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ inline int64_t first_lane64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// packed indices of one key block, as loaded (vector registers)
template <int NH, int NHV>
struct KeyIndices {
  int kb;
  int pk[NH];
  int pv[NHV];
  int pm, pb;
};

// Low half of a packed index.  Valid indices are below 2^31 (the block counts are), the marker of an
// inactive block is -1, so the low half carries everything the kernels test.
__device__ inline int low_half(const int64_t *p, int64_t i) { return reinterpret_cast<const int32_t *>(p)[2 * i]; }

template <int NH, int NHV>
__device__ inline KeyIndices<NH, NHV> load_key_indices(const bsa_attn_args &a, int64_t b, int64_t row, int kb) {
  KeyIndices<NH, NHV> r;
  r.kb = kb;
  const int64_t krow = b * a.nk + kb;
#pragma unroll
  for (int h = 0; h < NH; ++h) r.pk[h] = low_half(a.pidx_k, krow * NH + h);
#pragma unroll
  for (int h = 0; h < NHV; ++h) r.pv[h] = low_half(a.pidx_v, krow * NHV + h);
  r.pm = a.mask ? low_half(a.pidx_mask, row * a.nk + kb) : -1;
  r.pb = a.bias ? low_half(a.pidx_bias, row * a.nk + kb) : -1;
  return r;
}

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// Asynchronous copy of 64 x 16 bytes, global -> LDS: lane l's 16 bytes land at dst + 16 l (dst is wave
// uniform).  Completion is counted by vmcnt like any vector load.  Written as inline assembly so that the
// compiler's wait-count pass does not see it: it would otherwise wait for the copy in front of every later
// LDS read, also reads of other LDS arrays.  The caller waits (vmcnt(0)) before the data is read.  Copies
// the compiler does not know about only make the waits it computes for its own loads longer, never shorter.
__device__ inline void copy_1k_to_lds(const char *src, char *dst) {
  const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_ptr_t)dst;
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(src), "s"(lds_addr)
               : "memory", "m0");
}

template <typename Tr, int NH, int NHV>
__global__ __launch_bounds__(kFwdThreads, 2) void attn_fwd_mfma_kernel(bsa_attn_args a) {
  // two arrays, not one: the compiler then knows that the asynchronous K copy never touches the V tile
  __shared__ __attribute__((aligned(1024))) char lds_k[NH * kBlockBytes];
  __shared__ __attribute__((aligned(16))) char lds_v[NHV * kBlockBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = first_lane(tid >> 6);
  const int li = lane & 31, kg = lane >> 5;
  const int qi = 32 * wave + li;  // query row inside the block
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: give every XCD a contiguous
  // range of rows, so that the query blocks in flight on one L2 share their batch entry's K and V.
  const int64_t row = (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (row >= a.B * a.nq) return;
  const int64_t b = row / a.nq, qb = row % a.nq;
  const int k_begin = a.key_offsets[row], k_end = a.key_offsets[row + 1];

  // Q fragments stay in registers for the whole row
  u32x4 qf[NH][4];
#pragma unroll
  for (int h = 0; h < NH; ++h) {
    const int64_t pq = a.pidx_q[row * NH + h];
    const bool valid = pq >= 0 && pq < a.n_q_blocks;
    const char *qp = static_cast<const char *>(a.q) + (valid ? pq : 0) * kBlockBytes + qi * 128 + kg * 16;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      qf[h][s] = u32x4{0u, 0u, 0u, 0u};
      if (valid) qf[h][s] = *reinterpret_cast<const u32x4 *>(qp + 32 * s);
    }
  }

  f32x16 oacc[NHV][2];
#pragma unroll
  for (int h = 0; h < NHV; ++h)
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[h][db][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;

  const float qk_scale = a.scale * kLog2e;
  const bool causal = a.causal_lengths != nullptr;
  // positions fit 32 bits (the sequence block counts do); a longer length masks nothing more than INT_MAX does
  int seq_len = 0;
  if (causal) {
    const int64_t len = a.causal_lengths[b];
    seq_len = len < 0 ? 0 : (len > 0x7fffffffLL ? 0x7fffffff : (int)len);
  }
  const int qpos = (int)qb * kSbs + qi;

  if (k_begin < k_end) {
    u32x4 vr[NHV][4];  // staging registers of the V tile in flight
    uint32_t mask_nxt[8];
    // wave-uniform facts about the key block whose tiles are in flight
    int kb_nxt, pk_nxt[NH], pm_nxt, pb_nxt;

    // K tile: copied global -> LDS without passing through registers.  One instruction moves 1 KiB
    // (eight 128-byte rows); lane l supplies the 16-byte chunk that belongs at position l of that KiB,
    // which is where the XOR swizzle of the chunk index is applied.  Wave w copies rows 32 w .. 32 w + 31.
    auto copy_k = [&]() {
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        const int64_t pk = pk_nxt[h];
        if (pk >= 0) {
          const char *kp = static_cast<const char *>(a.k) + pk * kBlockBytes;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r0 = 32 * wave + 8 * i;
            const int r = r0 + (lane >> 3);
            const char *src = kp + r * 128 + (((lane & 7) ^ (r & 7)) << 4);
            copy_1k_to_lds(src, lds_k + h * kBlockBytes + r0 * 128);
          }
        } else {
          // inactive slice: zeros
#pragma unroll
          for (int i = 0; i < 4; ++i)
            *reinterpret_cast<u32x4 *>(lds_k + h * kBlockBytes + (i * kFwdThreads + tid) * 16) = u32x4{0u, 0u, 0u, 0u};
        }
      }
    };

    // facts and V tile of one key block
    auto fetch_v = [&](const KeyIndices<NH, NHV> &kx) {
      kb_nxt = first_lane(kx.kb);
#pragma unroll
      for (int h = 0; h < NH; ++h) {
        pk_nxt[h] = first_lane(kx.pk[h]);
        if (pk_nxt[h] >= a.n_k_blocks) pk_nxt[h] = -1;
      }
      pm_nxt = first_lane(kx.pm);
      if (pm_nxt >= a.n_mask_blocks) pm_nxt = -1;
      pb_nxt = first_lane(kx.pb);
      if (pb_nxt >= a.n_bias_blocks) pb_nxt = -1;
#pragma unroll
      for (int h = 0; h < NHV; ++h) {
        const int64_t pv = first_lane(kx.pv[h]);
        const bool valid = pv >= 0 && pv < a.n_v_blocks;
        const char *vp = static_cast<const char *>(a.v) + (valid ? pv : 0) * kBlockBytes;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int q = t * kFwdThreads + tid;
          const int ro = q & 7, jp = q >> 3;
          vr[h][2 * t] = u32x4{0u, 0u, 0u, 0u};
          vr[h][2 * t + 1] = u32x4{0u, 0u, 0u, 0u};
          if (valid) {
            vr[h][2 * t] = *reinterpret_cast<const u32x4 *>(vp + (2 * jp) * 128 + ro * 16);
            vr[h][2 * t + 1] = *reinterpret_cast<const u32x4 *>(vp + (2 * jp + 1) * 128 + ro * 16);
          }
        }
      }
    };

    // bytes j = 32 jb + 8 q + 4 kg .. + 3 of mask row qi: dword 16 qi + 8 jb + 2 q + kg
    auto fetch_mask = [&]() {
      if (pm_nxt >= 0) {
        const uint32_t *mp =
            static_cast<const uint32_t *>(a.mask) + (int64_t)pm_nxt * (kSbs * kSbs / 4) + qi * 16 + kg;
#pragma unroll
        for (int w = 0; w < 8; ++w) mask_nxt[w] = mp[2 * w];
      }
    };

    auto clamp_e = [&](int e) { return e < k_end ? e : k_end - 1; };

    // prologue of the three-stage index pipeline
    KeyIndices<NH, NHV> kx_nxt;
    int kbv_nn;
    {
      const int kb0 = a.key_indices[as_vector(k_begin)];
      const int kb1 = a.key_indices[as_vector(clamp_e(k_begin + 1))];
      kbv_nn = a.key_indices[as_vector(clamp_e(k_begin + 2))];
      const KeyIndices<NH, NHV> kx0 = load_key_indices<NH, NHV>(a, b, row, kb0);
      kx_nxt = load_key_indices<NH, NHV>(a, b, row, kb1);
      fetch_v(kx0);
      copy_k();
      fetch_mask();
    }

    for (int e = k_begin; e < k_end; ++e) {
      // ---- V tile e: registers -> LDS as (j, j+1) pairs; the K tile of e has been copied by now ----
#pragma unroll
      for (int h = 0; h < NHV; ++h)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int q = t * kFwdThreads + tid;
          const int ro = q & 7, jp = q >> 3;
          const u32x4 ev = vr[h][2 * t], od = vr[h][2 * t + 1];
          u32x4 lo, hi;
          lo[0] = __builtin_amdgcn_perm(od[0], ev[0], 0x05040100u);
          lo[1] = __builtin_amdgcn_perm(od[0], ev[0], 0x07060302u);
          lo[2] = __builtin_amdgcn_perm(od[1], ev[1], 0x05040100u);
          lo[3] = __builtin_amdgcn_perm(od[1], ev[1], 0x07060302u);
          hi[0] = __builtin_amdgcn_perm(od[2], ev[2], 0x05040100u);
          hi[1] = __builtin_amdgcn_perm(od[2], ev[2], 0x07060302u);
          hi[2] = __builtin_amdgcn_perm(od[3], ev[3], 0x05040100u);
          hi[3] = __builtin_amdgcn_perm(od[3], ev[3], 0x07060302u);
          uint32_t *prow = reinterpret_cast<uint32_t *>(lds_v + h * kBlockBytes) + jp * kSbs;
          *reinterpret_cast<u32x4 *>(prow + pair_col_offset(ro * 8)) = lo;
          *reinterpret_cast<u32x4 *>(prow + pair_col_offset(ro * 8 + 4)) = hi;
        }
      const bool mask_on = pm_nxt >= 0;
      const int kb = kb_nxt;
      const int64_t pb = pb_nxt;
      // mask words of tile e -> one bit per element (bit 4 w + t set: element masked); frees the word registers
      uint32_t mbits = 0;
      if (mask_on) {
#pragma unroll
        for (int w = 0; w < 8; ++w) {
          // bit 7 of a byte of z is set where the mask byte is zero (exact per byte: no borrow crosses bytes)
          const uint32_t x = mask_nxt[w];
          const uint32_t z = ~(((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
          // gather bits 7, 15, 23, 31 into a nibble
          const uint32_t nib = ((z >> 7) * 0x00204081u) >> 21 & 0xfu;
          mbits |= (nib ^ 0xfu) << (4 * w);
        }
      }
      // every outstanding copy of this wave (the K rows it moved) has to be in LDS before the barrier:
      // s_waitcnt vmcnt(0), other counters untouched
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();

      // ---- prefetch: V tile of e+1, packed indices of e+2, key index of e+3 ----
      const bool more = e + 1 < k_end;
      if (more) {
        fetch_v(kx_nxt);
        fetch_mask();
      }
      kx_nxt = load_key_indices<NH, NHV>(a, b, row, kbv_nn);
      kbv_nn = a.key_indices[as_vector(clamp_e(e + 3))];

      // A tile in which every score of this wave's 32 rows is masked changes nothing: m stays, alpha is 1,
      // every p is 0.  Such a tile is only fetched, not computed.
      bool live = true;
      if (mask_on) live = __any(mbits != 0xffffffffu);
      if (causal) {
        const int q_last = (int)qb * kSbs + 32 * wave + 31, q_first = q_last - 31;
        if (kb * kSbs > q_last || q_first >= seq_len || kb * kSbs >= seq_len) live = false;
      }

      // ---- S^T = K Q^T ----
      // Fragments are read from LDS in batches of four, one batch ahead of the MFMAs that consume them.
      f32x16 sacc[2];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[jb][r] = 0.f;
      if (live) {
        constexpr int kBatches = NH * 2;  // batch g: head slice g / 2, k steps 2 (g % 2) and 2 (g % 2) + 1, both key halves
        u32x4 kf[2][4];
        auto read_batch = [&](u32x4 (&dst)[4], int g) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int h = g >> 1, st = 2 * (g & 1) + (t >> 1), jb = t & 1;
            const int rj = 32 * jb + li;
            dst[t] = *reinterpret_cast<const u32x4 *>(lds_k + h * kBlockBytes + rj * 128 +
                                                      (((2 * st + kg) ^ (rj & 7)) << 4));
          }
        };
        read_batch(kf[0], 0);
#pragma unroll
        for (int g = 0; g < kBatches; ++g) {
          if (g + 1 < kBatches) read_batch(kf[(g + 1) & 1], g + 1);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int h = g >> 1, st = 2 * (g & 1) + (t >> 1), jb = t & 1;
            sacc[jb] = Tr::mfma(kf[g & 1][t], qf[h][st], sacc[jb]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }

      // both waves are done with the K tile of e: start the copy of the K tile of e+1 into its place
      __syncthreads();
      if (more) copy_k();

      if (live) {
      // first batch of V fragments: in flight while the softmax runs
      constexpr int kVBatches = NHV * 4;  // batch g: head slice g / 4, key quarter g % 4, both column halves
      u32x4 vf[2][2];
      auto read_vbatch = [&](u32x4 (&dst)[2], int g) {
        const int h = g >> 2, jq = g & 3;
#pragma unroll
        for (int db = 0; db < 2; ++db) {
          const uint32_t *vp = reinterpret_cast<const uint32_t *>(lds_v + h * kBlockBytes) +
                               pair_col_offset(32 * db + li) + (2 * kg + 8 * jq) * kSbs;
          dst[db][0] = vp[0];
          dst[db][1] = vp[kSbs];
          dst[db][2] = vp[4 * kSbs];
          dst[db][3] = vp[5 * kSbs];
        }
      };
      read_vbatch(vf[0], 0);
      __builtin_amdgcn_sched_barrier(0);

      // ---- scores: scale, bias, causal predicate, mask ----
      float sv[32];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[16 * jb + r] = sacc[jb][r] * qk_scale;
      if (pb >= 0) {
        // bias elements j = 32 jb + 8 q + 4 kg .. + 3 of row qi
        const char *bp = static_cast<const char *>(a.bias) + pb * kBlockBytes + qi * 128 + kg * 8;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
          const u32x2 bw = *reinterpret_cast<const u32x2 *>(bp + 16 * w);
          sv[4 * w + 0] += Tr::widen((uint16_t)(bw[0] & 0xffffu)) * kLog2e;
          sv[4 * w + 1] += Tr::widen((uint16_t)(bw[0] >> 16)) * kLog2e;
          sv[4 * w + 2] += Tr::widen((uint16_t)(bw[1] & 0xffffu)) * kLog2e;
          sv[4 * w + 3] += Tr::widen((uint16_t)(bw[1] >> 16)) * kLog2e;
        }
      }
      if (causal) {
        const int kbase = kb * kSbs + 4 * kg;
        const bool row_off = qpos >= seq_len;
#pragma unroll
        for (int w = 0; w < 8; ++w)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int kpos = kbase + 8 * w + t;
            if (kpos > qpos || row_off || kpos >= seq_len) sv[4 * w + t] = -INFINITY;
          }
      }
      if (mask_on) {
        // most blocks of a mask mask nothing: one test for the wave skips the selects
        if (__any(mbits != 0)) {
#pragma unroll
          for (int x = 0; x < 32; ++x) sv[x] = ((mbits >> x) & 1u) ? -INFINITY : sv[x];
        }
      }

      // ---- online softmax of row qi ----
      float m_blk = sv[0];
#pragma unroll
      for (int x = 1; x < 32; ++x) m_blk = fmaxf(m_blk, sv[x]);
      m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32));
      const float m_new = fmaxf(m_i, m_blk);
      const bool both_ninf = (m_i == -INFINITY) && (m_new == -INFINITY);
      const float alpha = both_ninf ? 1.f : __builtin_amdgcn_exp2f(m_i - m_new);
      // with m_new == -inf every score of the row is -inf (or NaN): subtracting 0 instead keeps p = 0
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;
      float sum = 0.f;
#pragma unroll
      for (int x = 0; x < 32; ++x) {
        sv[x] = __builtin_amdgcn_exp2f(sv[x] - m_sub);
        sum += sv[x];
      }
      sum += __shfl_xor(sum, 32);
      l_i = l_i * alpha + sum;
      m_i = m_new;

      u32x4 pf[2][2];
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int t = 0; t < 4; ++t)
            pf[jb][u][t] = Tr::pack2(sv[16 * jb + 8 * u + 2 * t], sv[16 * jb + 8 * u + 2 * t + 1]);

      // ---- O^T = alpha O^T + V^T P^T ----
      // once the running maximum has settled alpha is 1 for every row of the wave
      if (__any(alpha != 1.f)) {
#pragma unroll
        for (int h = 0; h < NHV; ++h)
#pragma unroll
          for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[h][db][r] *= alpha;
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int g = 0; g < kVBatches; ++g) {
        if (g + 1 < kVBatches) read_vbatch(vf[(g + 1) & 1], g + 1);
        __builtin_amdgcn_sched_barrier(0);
        const int h = g >> 2, jq = g & 3;
#pragma unroll
        for (int db = 0; db < 2; ++db) oacc[h][db] = Tr::mfma(vf[g & 1][db], pf[jq >> 1][jq & 1], oacc[h][db]);
        __builtin_amdgcn_sched_barrier(0);
      }
      }  // live
      __syncthreads();
    }
  }

  // ---- epilogue: O = O^T^T / l, lse = m + log2(l) ----
#pragma unroll
  for (int h = 0; h < NHV; ++h) {
    const int64_t po = a.pidx_o[row * NHV + h];
    if (po < 0 || po >= a.n_o_blocks) continue;
    char *op = static_cast<char *>(a.o) + po * kBlockBytes + qi * 128 + kg * 8;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = (l_i != 0.f) ? oacc[h][db][4 * q + t] / l_i : 0.f;
        u32x2 w;
        w[0] = Tr::pack2(v[0], v[1]);
        w[1] = Tr::pack2(v[2], v[3]);
        *reinterpret_cast<u32x2 *>(op + 64 * db + 16 * q) = w;
      }
  }
  if (kg == 0) a.lse[row * kSbs + qi] = (l_i != 0.f) ? m_i + log2f(l_i) : -INFINITY;
}

template <typename Tr, int NH, int NHV>
int launch_fwd(const bsa_attn_args &a, hipStream_t s) {
  const int64_t rows = a.B * a.nq;
  if (rows == 0) return BSA_OK;
  attn_fwd_mfma_kernel<Tr, NH, NHV><<<(unsigned)(cdiv(rows, 8) * 8), kFwdThreads, 0, s>>>(a);
  return check_launch("attn_fwd_mfma_kernel");
}

template <typename Tr>
int dispatch_fwd(const bsa_attn_args &a, hipStream_t s) {
  if (a.nh == 1 && a.nhv == 1) return launch_fwd<Tr, 1, 1>(a, s);
  if (a.nh == 2 && a.nhv == 2) return launch_fwd<Tr, 2, 2>(a, s);
  if (a.nh == 1 && a.nhv == 2) return launch_fwd<Tr, 1, 2>(a, s);
  if (a.nh == 2 && a.nhv == 1) return launch_fwd<Tr, 2, 1>(a, s);
  return 1;
}

}  // namespace

int attn_fwd_mfma(const bsa_attn_args &a, hipStream_t s) {
  if (a.sbs != kSbs || (a.dtype != BSA_BF16 && a.dtype != BSA_F16)) return 1;
  // a query row without key_indices (an attention layout without active blocks) still writes o and lse
  if (a.key_indices == nullptr && a.B * a.nq > 0) return 1;
  return a.dtype == BSA_BF16 ? dispatch_fwd<MBf16>(a, s) : dispatch_fwd<MF16>(a, s);
}

int attn_bwd_mfma(const bsa_attn_args &, hipStream_t) { return 1; }

}  // namespace bsa
