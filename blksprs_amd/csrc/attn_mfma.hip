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
// fragment is gathered from LDS for exactly that key set.  K and V are both kept
// row-major in LDS with XOR-swizzled 16-byte chunks: a K fragment (head dimension
// contracted) is one 128-bit read, a V fragment (key index contracted) is two
// transposing 64-bit reads (ds_read_b64_tr_b16), so neither tile passes through registers.
//
// The K / V tiles of key block e+1, the mask words of e+1, the packed indices of e+2
// and the key index of e+3 are all fetched while block e is computed.  The index
// fetches are one vector load (each index in its own lane) on purpose: it completes
// in order with the tile loads, so the one wait at the top of an iteration covers it
// and no scalar-load wait lands in front of an LDS read.  The vector memory pipeline
// works per instruction, so the count of load instructions per tile is kept small.
//
// Score pipeline (log2 domain), in this order: scale * q k^T, + bias, native causal
// predicate, explicit mask; probabilities are rounded to the operand type before they
// multiply V; the row sum uses the unrounded values.
#include "attn_mfma_common.h"

namespace bsa {
namespace {

using namespace mfma;

constexpr int kFwdThreads = 256;
constexpr float kRescaleStep = 8.f;  // log2 units

// One workgroup (four waves) owns a PAIR of neighbouring query blocks and walks the union of their key lists,
// so that a K / V tile both of them need is fetched once; bits 28 and 29 of a list entry say which of the
// two the key block is active for.  Waves 0, 1 own the first query block, waves 2, 3 the second.
//
// The K and V tiles are double buffered in LDS: while tile e is computed from one buffer, the K tile of e+1 is
// copied into the other and the V tile of e+1 travels through registers into it; ONE barrier per tile, at
// its end, says both that the next tile is complete and that this one's buffer may be overwritten.
template <typename Tr, int NH, int NHV>
__global__ __launch_bounds__(kFwdThreads, 2) void attn_fwd_mfma_kernel(bsa_attn_args a) {
  constexpr int G = 2;
  constexpr int kThreads = kFwdThreads;
  constexpr int kKBytes = NH * kBlockBytes, kVBytes = NHV * kBlockBytes;
  // two arrays, not one: the compiler then knows that the asynchronous K copy never touches the V tiles
  __shared__ __attribute__((aligned(1024))) char lds_k[2 * kKBytes];
  __shared__ __attribute__((aligned(16))) char lds_v[2 * kVBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = first_lane(tid >> 6);
  const int li = lane & 31, kg = lane >> 5;
  const int qi = 32 * (wave & 1) + li;  // query row inside the block
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: give every XCD a contiguous
  // range of groups, so that the query blocks in flight on one L2 share their batch entry's K and V.
  const int64_t groups_per_batch = (a.nq + G - 1) / G;
  const int64_t grp = (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (grp >= a.B * groups_per_batch) return;
  const int64_t b = grp / groups_per_batch;
  const int64_t qb_raw = (grp % groups_per_batch) * G + (wave >> 1);
  // a group at the end of an odd sequence has one query block only: its second pair of waves only helps to copy
  const bool has_q = qb_raw < a.nq;
  const int64_t qb = has_q ? qb_raw : a.nq - 1;
  const int64_t row = b * a.nq + qb;
  const AttnFwdRecord *recs = reinterpret_cast<const AttnFwdRecord *>(a.group_records);
  const int k_begin = a.group_offsets[grp], k_end = a.group_offsets[grp + 1];
  const int my_bit = 28 + (wave >> 1);

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
    u32x4 mask_a[2], mask_b[2];  // mask words of a tile as loaded: a = arrived, being judged; b = in flight
    // Per-tile facts travel through a short pipeline.  For tile j: its record is loaded while tile j-3 is
    // computed, its mask words while j-2 is computed; at the end of j-2 every wave says whether the tile is
    // dead for it (nothing of its 32 rows survives the mask, or its query block does not have the key block),
    // and only a tile that is live for some wave is copied to LDS while j-1 is computed.
    struct Facts {
      int entry, pm, pb;    // list entry, mask block, bias block (of this wave's query block)
      uint32_t mbits;       // per lane: mask of its 32 scores of the tile, bit 8 t + w = byte t of word w
      bool dead;            // for this wave
    };
    __shared__ int dead_votes[2][4];

    // K and V tiles: copied global -> LDS without passing through registers.  One instruction moves 1 KiB
    // (eight 128-byte rows); lane l supplies the 16-byte chunk that belongs at position l of that KiB, which
    // is where the XOR swizzle of the chunk index is applied (it depends on row % 8 only, so both KiB of a
    // wave's 16 rows use the same lane offsets).  Wave w copies rows 16 w .. 16 w + 15 of every slice.
    const uint32_t copy_off = (uint32_t)(16 * wave + (lane >> 3)) * 128u + (uint32_t)(((lane & 7) ^ t_swizzle(lane >> 3)) << 4);
    const uint32_t n_k32 = (uint32_t)(a.n_k_blocks < 0x7fffffffLL ? a.n_k_blocks : 0x7fffffffLL);
    const uint32_t n_v32 = (uint32_t)(a.n_v_blocks < 0x7fffffffLL ? a.n_v_blocks : 0x7fffffffLL);
    auto copy_slice = [&](const void *tensor, int32_t idx, uint32_t n_blocks, char *dst) {
      if ((uint32_t)idx < n_blocks) {  // also false for -1 (no such block)
        copy_2k_to_lds(static_cast<const char *>(tensor) + ((uint64_t)(uint32_t)idx << 13), copy_off, dst + wave * 2048);
      } else {
        // inactive slice: zeros
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<u32x4 *>(dst + (i * kThreads + tid) * 16) = u32x4{0u, 0u, 0u, 0u};
      }
    };
    auto copy_k = [&](const AttnFwdRecord &r, int buf) {
#pragma unroll
      for (int h = 0; h < NH; ++h) copy_slice(a.k, r.pk[h], n_k32, lds_k + buf * kKBytes + h * kBlockBytes);
    };

    // facts of one key block (without the mask, which arrives later)
    auto make_facts = [&](const AttnFwdRecord &r) {
      Facts f;
      f.entry = r.entry;
      f.pm = a.mask ? ((wave >> 1) ? r.pm[1] : r.pm[0]) : -1;
      if (f.pm >= a.n_mask_blocks) f.pm = -1;
      f.pb = a.bias ? ((wave >> 1) ? r.pb[1] : r.pb[0]) : -1;
      if (f.pb >= a.n_bias_blocks) f.pb = -1;
      f.mbits = 0;
      f.dead = false;
      return f;
    };

    // V tile: copied like the K tile; its rows become matrix-core operands through the transposing LDS load
    auto copy_v = [&](const AttnFwdRecord &r, int buf) {
#pragma unroll
      for (int h = 0; h < NHV; ++h) copy_slice(a.v, r.pv[h], n_v32, lds_v + buf * kVBytes + h * kBlockBytes);
    };

    // Mask words of the tile: lane (li, kg) needs bytes j = 32 jb + 8 q + 4 kg .. + 3 of mask row qi, that is
    // dword 8 jb + 2 q + kg of the row, as word 4 jb + q.  It loads the 32 bytes [32 kg, 32 kg + 32) of the
    // row (two 16-byte loads; the wave reads 2 KiB contiguously) and trades every other dword with lane
    // (li, 1 - kg): one swap of the upper half of a register with the lower half of another per q.
    auto fetch_mask = [&](int pm, u32x4 (&mask_raw)[2]) {
      if (pm >= 0) {
        const char *mp = static_cast<const char *>(a.mask) + (int64_t)pm * (kSbs * kSbs);
        const uint32_t moff = (uint32_t)qi * 64u + (uint32_t)kg * 32u;
        mask_raw[0] = load16(mp, moff);
        mask_raw[1] = load16(mp + 16, moff);
      }
    };
    auto mask_word = [&](const u32x4 (&mask_raw)[2], int w) -> uint32_t {
      // w = 4 jb + q: after the swap of (dword 2q, dword 2q + 1) the first holds the word of jb = 0, the second of jb = 1
      const int q = w & 3;
      const u32x2 sw = __builtin_amdgcn_permlane32_swap(mask_raw[q >> 1][2 * (q & 1)], mask_raw[q >> 1][2 * (q & 1) + 1],
                                                        false, false);
      return sw[w >> 2];
    };

    // mask words (bytes 0 or 1) -> one bit per score, then this wave's verdict on the tile
    auto finish_facts = [&](Facts &f, const u32x4 (&mask_raw)[2]) {
      f.mbits = 0;
      if (f.pm >= 0) {
#pragma unroll
        for (int w = 0; w < 8; ++w) f.mbits |= mask_word(mask_raw, w) << w;
      }
      bool live = has_q && ((f.entry >> my_bit) & 1);
      if (f.pm >= 0 && live) live = __any(f.mbits != 0xffffffffu);
      if (causal) {
        const int kb = f.entry & 0x0fffffff;
        const int q_last = (int)qb * kSbs + 32 * (wave & 1) + 31, q_first = q_last - 31;
        if (kb * kSbs > q_last || q_first >= seq_len || kb * kSbs >= seq_len) live = false;
      }
      f.dead = !live;
    };
    // without a mask or a causal predicate some wave always has work on a tile
    const bool may_skip = a.mask != nullptr || causal;
    auto vote = [&](const Facts &f, int pos) {
      if (may_skip && lane == 0) dead_votes[pos & 1][wave] = f.dead ? 1 : 0;
    };
    auto all_dead = [&](int pos) {
      if (!may_skip) return false;
      const int *v = dead_votes[pos & 1];
      return first_lane(v[0] & v[1] & v[2] & v[3]) != 0;
    };

    auto clamp_e = [&](int e) { return e < k_end ? e : k_end - 1; };

    // The record of a list entry (key block, packed indices of its K / V / mask / bias blocks) is read two
    // tiles before its tile is used, by ONE vector load (field i in lane i): that load completes in order with
    // the tile loads, so the wait at the end of a tile covers it, whereas a scalar load would put its full
    // latency in front of the next LDS read.  rv_next is the record of the tile after the current one.
    auto load_record = [&](int pos) -> int {
      int v = 0;
      if (lane < 9) v = reinterpret_cast<const int32_t *>(recs + pos)[lane];
      return v;
    };
    auto unpack_record = [&](int rv) {
      AttnFwdRecord r;
      r.entry = __builtin_amdgcn_readlane(rv, 0);
      r.pk[0] = __builtin_amdgcn_readlane(rv, 1);
      r.pk[1] = __builtin_amdgcn_readlane(rv, 2);
      r.pv[0] = __builtin_amdgcn_readlane(rv, 3);
      r.pv[1] = __builtin_amdgcn_readlane(rv, 4);
      r.pm[0] = __builtin_amdgcn_readlane(rv, 5);
      r.pm[1] = __builtin_amdgcn_readlane(rv, 6);
      r.pb[0] = __builtin_amdgcn_readlane(rv, 7);
      r.pb[1] = __builtin_amdgcn_readlane(rv, 8);
      return r;
    };
    // prologue: tile k_begin copied and judged, tile k_begin + 1 judged, mask words of k_begin + 2 and the
    // record of k_begin + 3 in flight
    Facts f0, f1, f2;
    AttnFwdRecord r1, r2;
    int rv3;
    {
      const AttnFwdRecord r0 = unpack_record(load_record(k_begin));
      const int rv1 = load_record(clamp_e(k_begin + 1));
      const int rv2 = load_record(clamp_e(k_begin + 2));
      rv3 = load_record(clamp_e(k_begin + 3));
      f0 = make_facts(r0);
      copy_k(r0, 0);
      copy_v(r0, 0);
      fetch_mask(f0.pm, mask_a);
      r1 = unpack_record(rv1);
      f1 = make_facts(r1);
      finish_facts(f0, mask_a);
      fetch_mask(f1.pm, mask_a);
      r2 = unpack_record(rv2);
      f2 = make_facts(r2);
      finish_facts(f1, mask_a);
      vote(f1, k_begin + 1);
      fetch_mask(f2.pm, mask_b);
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the rows this wave copied are in LDS
      __syncthreads();
    }

    for (int e = k_begin; e < k_end; ++e) {
      const int buf = (e - k_begin) & 1;
      // mask words of tile e+2, requested one tile ago
      mask_a[0] = mask_b[0];
      mask_a[1] = mask_b[1];
      // tile e+1: copied unless no wave has anything to compute on it.  Issued before this tile's other loads, so
      // that the wait at the end of the tile can leave those outstanding.
      const bool more = e + 1 < k_end;
      if (more && !all_dead(e + 1)) {
        copy_k(r1, buf ^ 1);
        copy_v(r1, buf ^ 1);
      }
      // tile e+3: facts from its record, mask words requested; record of tile e+4 requested
      const AttnFwdRecord r3 = unpack_record(rv3);
      Facts f3 = make_facts(r3);
      const int rv4 = load_record(clamp_e(e + 4));
      fetch_mask(f3.pm, mask_b);

      // tile e.  A tile in which every score of this wave's 32 rows is masked changes nothing: m stays, alpha
      // is 1, every p is 0.
      const bool mask_on = f0.pm >= 0;
      const int kb = f0.entry & 0x0fffffff;
      const int64_t pb = f0.pb;
      const uint32_t mbits = f0.mbits;
      const bool live = !f0.dead;

      if (live) {
        const char *kbuf = lds_k + buf * kKBytes;
        const char *vbuf = lds_v + buf * kVBytes;
        // ---- S^T = K Q^T ----
        // Fragments are read from LDS in batches of four, one batch ahead of the MFMAs that consume them.
        f32x16 sacc[2];
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[jb][r] = 0.f;
        {
          constexpr int kBatches = NH * 2;  // batch g: head slice g / 2, k steps 2 (g % 2), 2 (g % 2) + 1, both key halves
          u32x4 kf[2][4];
          auto read_batch = [&](u32x4 (&dst)[4], int g) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int h = g >> 1, st = 2 * (g & 1) + (t >> 1), jb = t & 1;
              const int rj = 32 * jb + li;
              dst[t] = *reinterpret_cast<const u32x4 *>(kbuf + h * kBlockBytes + rj * 128 +
                                                        (((2 * st + kg) ^ t_swizzle(rj)) << 4));
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

        // first batch of V fragments: in flight while the softmax runs
        constexpr int kVBatches = NHV * 4;  // batch g: head slice g / 4, key quarter g % 4, both column halves
        u32x4 vf[2][2];
        auto read_vbatch = [&](u32x4 (&dst)[2], int g) {
          const int h = g >> 2, jq = g & 3;
#pragma unroll
          for (int db = 0; db < 2; ++db)
            // keys 16 jq + 4 kg .. + 3 and + 8 .. + 11, column 32 db + lane % 32
            dst[db] = frag_cols_t(vbuf + h * kBlockBytes, 16 * jq + 4 * kg, 32 * db + 16 * ((lane >> 4) & 1), lane);
        };
        read_vbatch(vf[0], 0);
        __builtin_amdgcn_sched_barrier(0);

        // ---- scores: scale, bias, causal predicate, mask ----
        // sv holds the scores up to the positive factor cc: the raw dot products (cc = scale * log2 e), or, with
        // a bias, the finished log2-domain scores (cc = 1).  The factor is applied inside the exponential.
        float sv[32];
        float cc = qk_scale;
  #pragma unroll
        for (int jb = 0; jb < 2; ++jb)
  #pragma unroll
          for (int r = 0; r < 16; ++r) sv[16 * jb + r] = sacc[jb][r];
        if (pb >= 0) {
          // bias elements j = 32 jb + 8 q + 4 kg .. + 3 of row qi
          const char *bp0 = static_cast<const char *>(a.bias) + pb * kBlockBytes;
          const uint32_t boff = (uint32_t)qi * 128u + (uint32_t)kg * 8u;
  #pragma unroll
          for (int w0 = 0; w0 < 8; w0 += 2) {
            u32x2 bw[2];
  #pragma unroll
            for (int w = 0; w < 2; ++w) bw[w] = *reinterpret_cast<const u32x2 *>(bp0 + 16 * (w0 + w) + boff);
  #pragma unroll
            for (int w = 0; w < 2; ++w) {
              float *d = sv + 4 * (w0 + w);
              d[0] = d[0] * qk_scale + Tr::widen((uint16_t)(bw[w][0] & 0xffffu)) * kLog2e;
              d[1] = d[1] * qk_scale + Tr::widen((uint16_t)(bw[w][0] >> 16)) * kLog2e;
              d[2] = d[2] * qk_scale + Tr::widen((uint16_t)(bw[w][1] & 0xffffu)) * kLog2e;
              d[3] = d[3] * qk_scale + Tr::widen((uint16_t)(bw[w][1] >> 16)) * kLog2e;
            }
          }
          cc = 1.f;
        }
        // most tiles lie where the predicate holds for every score of the wave's 32 rows (every key of the tile at or
        // before the wave's first query, and the wave's last query inside the sequence): one test for the wave
        // skips the selects
        const int q_wave_first = (int)qb * kSbs + 32 * (wave & 1);
        if (causal && (kb * kSbs + kSbs - 1 > q_wave_first || q_wave_first + 31 >= seq_len)) {
          const int kbase = kb * kSbs + 4 * kg;
          const bool row_off = qpos >= seq_len;
  #pragma unroll
          for (int w = 0; w < 8; ++w)
  #pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int kpos = kbase + 8 * w + t;
              sv[4 * w + t] = (kpos > qpos || row_off || kpos >= seq_len) ? -INFINITY : sv[4 * w + t];
            }
        }
        if (mask_on) {
          // most blocks of a mask mask nothing: one test for the wave skips the selects
          if (__any(mbits != 0)) {
  #pragma unroll
            for (int x = 0; x < 32; ++x) sv[x] = ((mbits >> (8 * (x & 3) + (x >> 2))) & 1u) ? -INFINITY : sv[x];
          }
        }

        // ---- online softmax of row qi ----
        float m_blk = sv[0];
  #pragma unroll
        for (int x = 1; x < 32; ++x) m_blk = fmaxf(m_blk, sv[x]);
        m_blk = max_across32(m_blk) * cc;
        // The reference maximum m_i of the exponentials only follows the running maximum when that has grown by
        // more than kRescaleStep since the last update (for some row of the wave): in between, probabilities may
        // exceed 1 (by at most 2^kRescaleStep) and the accumulators need no rescaling.  o and lse do not depend on
        // the reference maximum.  -inf - -inf is NaN and compares false: a row without a finite score keeps -inf.
        const float m_cand = fmaxf(m_i, m_blk);
        if (__any((m_cand - m_i) > kRescaleStep)) {
          const bool both_ninf = (m_i == -INFINITY) && (m_cand == -INFINITY);
          const float alpha = both_ninf ? 1.f : __builtin_amdgcn_exp2f(m_i - m_cand);
          m_i = m_cand;
          l_i *= alpha;
  #pragma unroll
          for (int h = 0; h < NHV; ++h)
  #pragma unroll
            for (int db = 0; db < 2; ++db)
  #pragma unroll
              for (int r = 0; r < 16; ++r) oacc[h][db][r] *= alpha;
        }
        // with m_i == -inf every score of the row so far is -inf (or NaN): subtracting 0 instead keeps p = 0
        const float m_sub = (m_i == -INFINITY) ? 0.f : m_i;
        float sum = 0.f;
  #pragma unroll
        for (int x = 0; x < 32; ++x) {
          sv[x] = __builtin_amdgcn_exp2f(fmaf(sv[x], cc, -m_sub));
          sum += sv[x];
        }
        l_i += sum;  // of this lane's 32 keys: the two halves of a row are added once, in the epilogue

        u32x4 pf[2][2];
  #pragma unroll
        for (int jb = 0; jb < 2; ++jb)
  #pragma unroll
          for (int u = 0; u < 2; ++u)
  #pragma unroll
            for (int t = 0; t < 4; ++t)
              pf[jb][u][t] = Tr::pack2(sv[16 * jb + 8 * u + 2 * t], sv[16 * jb + 8 * u + 2 * t + 1]);

        // ---- O^T += V^T P^T ----
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

      // ---- the barrier ends the reads of tile e and publishes tile e+1 and the verdicts on tile e+2 ----
      finish_facts(f2, mask_a);
      vote(f2, e + 2);
      // The rows this wave copied have to be in LDS; the loads issued after the copies (a record, two mask
      // loads if the tile has a mask block) may stay in flight.  vmcnt(3) / vmcnt(1), other counters untouched.
      // The counts follow this iteration's issue order at the top of the loop: copy_k / copy_v (the asynchronous
      // copies of tile e + 1), then load_record (one vector load, the record of tile e + 4), then fetch_mask,
      // which issues two loads only when the record of tile e + 3 names a mask block (f3.pm >= 0).  vmcnt
      // retires in issue order, so "at most 1 (3) outstanding" leaves exactly those younger loads in flight.
      // The bias loads of the tile are consumed (and so waited for by the compiler) inside the tile.  A load
      // added after the copies and not consumed before this point would make these waits too lax by one: it has
      // to be added to both counts.
      if (f3.pm >= 0) __builtin_amdgcn_s_waitcnt(0x0F73);
      else __builtin_amdgcn_s_waitcnt(0x0F71);
      f0 = f1;
      f1 = f2;
      f2 = f3;
      r1 = r2;
      r2 = r3;
      rv3 = rv4;
      __syncthreads();
    }
  }

  // ---- epilogue: O = O^T^T / l, lse = m + log2(l) ----
  if (!has_q) return;
  // one reciprocal per row, then products: 64 IEEE divisions per lane cost ten instructions each, and the last
  // bit they would buy is rounded away with the other fifteen when the quotient becomes a 16-bit value
  l_i = sum_across32(l_i);
  const float inv_l = (l_i != 0.f) ? 1.f / l_i : 0.f;
  // A lane holds eight bytes of a row at a time (register 4 q + t of half db: column 32 db + 8 q + 4 kg + t).  The
  // wave writes its 32 rounded rows into LDS (the V tiles are free: every wave has passed the last tile's barrier),
  // 128 bytes per row with the 16-byte chunks swizzled by the row, and stores them from there, eight lanes to a
  // row: whole lines per instruction, past the caches.  Rows and chunks are the wave's own, so no barrier.
  char *rows_lds = lds_v + (wave >> 1) * NHV * kBlockBytes;
#pragma unroll
  for (int h = 0; h < NHV; ++h)
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) v[t] = oacc[h][db][4 * q + t] * inv_l;
        u32x2 w;
        w[0] = Tr::pack2(v[0], v[1]);
        w[1] = Tr::pack2(v[2], v[3]);
        *reinterpret_cast<u32x2 *>(rows_lds + h * kBlockBytes + qi * 128 + (((4 * db + q) ^ (qi & 7)) << 4) + 8 * kg) = w;
      }
#pragma unroll
  for (int h = 0; h < NHV; ++h) {
    const int64_t po = a.pidx_o[row * NHV + h];
    if (po < 0 || po >= a.n_o_blocks) continue;
    char *out = static_cast<char *>(a.o) + po * kBlockBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 32 * (wave & 1) + 8 * i + (lane >> 3), c = lane & 7;
      const u32x4 v = *reinterpret_cast<const u32x4 *>(rows_lds + h * kBlockBytes + r * 128 + ((c ^ (r & 7)) << 4));
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(out + r * 128 + c * 16));
    }
  }
  if (kg == 0) a.lse[row * kSbs + qi] = (l_i != 0.f) ? m_i + log2f(l_i) : -INFINITY;
}

// One workgroup per group of query blocks: expands the group's list entries into records.
__global__ __launch_bounds__(64) void attn_fwd_records_kernel(bsa_attn_args a, const int32_t *entries,
                                                              AttnFwdRecord *records) {
  const int64_t grp = blockIdx.x;
  const int G = a.group_size;
  const int64_t groups_per_batch = (a.nq + G - 1) / G;
  const int64_t b = grp / groups_per_batch, q0 = (grp % groups_per_batch) * G;
  const int begin = a.group_offsets[grp], end = a.group_offsets[grp + 1];
  for (int e = begin + (int)threadIdx.x; e < end; e += 64) {
    const int32_t ent = entries[e];
    const int64_t kb = ent & 0x0fffffff;
    AttnFwdRecord r;
    r.entry = ent;
    for (int h = 0; h < 2; ++h) {
      r.pk[h] = h < a.nh ? (int32_t)a.pidx_k[(b * a.nk + kb) * a.nh + h] : -1;
      r.pv[h] = h < a.nhv ? (int32_t)a.pidx_v[(b * a.nk + kb) * a.nhv + h] : -1;
    }
    for (int g = 0; g < 2; ++g) {
      const int64_t qb = q0 + g;
      const bool has = g < G && qb < a.nq && ((ent >> (28 + g)) & 1);
      const int64_t pair = (b * a.nq + qb) * a.nk + kb;
      r.pm[g] = has && a.pidx_mask ? (int32_t)a.pidx_mask[pair] : -1;
      r.pb[g] = has && a.pidx_bias ? (int32_t)a.pidx_bias[pair] : -1;
    }
    for (int i = 0; i < 7; ++i) r.pad[i] = 0;
    records[e] = r;
  }
}

template <typename Tr, int NH, int NHV>
int launch_fwd(const bsa_attn_args &a, hipStream_t s) {
  const int64_t groups = a.B * cdiv(a.nq, 2);
  if (groups == 0) return BSA_OK;
  attn_fwd_mfma_kernel<Tr, NH, NHV><<<(unsigned)(cdiv(groups, 8) * 8), kFwdThreads, 0, s>>>(a);
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
  // the kernels take the row maximum before the scale is applied
  if (!(a.scale > 0.f) || a.scale > 3.0e38f) return 1;
  // the matrix-core kernels walk the grouped record lists; without them the generic kernels run
  if (a.group_offsets == nullptr || a.group_size != 2) return 1;
  if (a.group_records == nullptr) {
    // no list entry at all: every query block still writes o = 0 and lse = -inf
    // (the caller passes NULL for an empty record array; the offsets then are all zero)
  }
  return a.dtype == BSA_BF16 ? dispatch_fwd<MBf16>(a, s) : dispatch_fwd<MF16>(a, s);
}

int attn_fwd_records(const bsa_attn_args &a, const int32_t *entries, int32_t *records, hipStream_t s) {
  const int64_t groups = a.B * cdiv(a.nq, a.group_size);
  if (groups == 0) return BSA_OK;
  attn_fwd_records_kernel<<<(unsigned)groups, 64, 0, s>>>(a, entries, reinterpret_cast<AttnFwdRecord *>(records));
  return check_launch("attn_fwd_records_kernel");
}


}  // namespace bsa
