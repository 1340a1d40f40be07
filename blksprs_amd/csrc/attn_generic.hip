// Block-sparse flash attention, generic kernels: any of fp32 / fp16 / bf16, sbs in {16, 32, 64},
// any number of head slices, fp32 FMA arithmetic on LDS tiles.
//
// These cover the configurations the MFMA kernels do not and are written for
// clarity of the semantics, not speed.  One workgroup owns one (batch, sequence
// block, head slice): the score tile of a (query block, key block) pair is
// recomputed for every head slice, which keeps every accumulator in registers and
// leaves no read-modify-write of global memory and no atomics.
//
// Score pipeline (log2 domain), in this order: scale * q k^T, + bias, native causal
// predicate, explicit mask.  Probabilities are rounded to the operand type before
// they multiply V (forward) or dO (backward); ds likewise before it multiplies Q / K.
#include "attn_common.h"

namespace bsa {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxOwn = 16;  // 64*64 / 256 tile elements per thread

struct Tiles {
  float *a;  // [sbs][sbs + 1]
  float *b;  // [sbs][sbs + 1]
  float *s;  // [sbs][sbs + 1]
};

// Cooperative load of one sbs x sbs block into LDS as fp32; transpose stores element (r, c) at [c][r].
template <typename Tr>
__device__ inline void load_block(float *dst, const typename Tr::elem_t *blk, int sbs, bool transpose) {
  const int ld = sbs + 1;
  for (int idx = threadIdx.x; idx < sbs * sbs; idx += kThreads) {
    const int r = idx / sbs, c = idx % sbs;
    const float v = Tr::widen(blk[idx]);
    if (transpose) dst[c * ld + r] = v; else dst[r * ld + c] = v;
  }
}

// acc[m] += sum_d A[i][d] * Bt[d][j] for the elements (i, j) this thread owns
__device__ inline void tile_mac(float (&acc)[kMaxOwn], const float *A, const float *Bt, int sbs) {
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      const int i = idx / sbs, j = idx % sbs;
      float v = acc[m];
      for (int d = 0; d < sbs; ++d) v = fmaf(A[i * ld + d], Bt[d * ld + j], v);
      acc[m] = v;
    }
  }
}

// Scores of (query block qb, key block kb) of batch b into t.s, log2 domain, with bias, causal predicate and mask.
template <typename Tr>
__device__ inline void score_tile(const bsa_attn_args &a, const Tiles &t, int64_t b, int64_t qb, int64_t kb) {
  using E = typename Tr::elem_t;
  const int sbs = a.sbs;
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
  float acc[kMaxOwn];
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) acc[m] = 0.f;
  for (int64_t h = 0; h < a.nh; ++h) {
    const int64_t pq = a.pidx_q[(b * a.nq + qb) * a.nh + h];
    const int64_t pk = a.pidx_k[(b * a.nk + kb) * a.nh + h];
    if (pq < 0 || pk < 0 || pq >= a.n_q_blocks || pk >= a.n_k_blocks) continue;
    __syncthreads();
    load_block<Tr>(t.a, static_cast<const E *>(a.q) + pq * sbs * sbs, sbs, false);
    load_block<Tr>(t.b, static_cast<const E *>(a.k) + pk * sbs * sbs, sbs, true);
    __syncthreads();
    tile_mac(acc, t.a, t.b, sbs);
  }
  const float qk_scale = a.scale * kLog2e;
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
  const bool causal = a.causal_lengths != nullptr;
  const int64_t len = causal ? a.causal_lengths[b] : 0;
  __syncthreads();
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      const int i = idx / sbs, j = idx % sbs;
      float s = acc[m] * qk_scale;
      if (pb >= 0) s = s + Tr::widen(static_cast<const E *>(a.bias)[pb * sbs * sbs + idx]) * kLog2e;
      if (causal) {
        const int64_t qp = qb * sbs + i, kp = kb * sbs + j;
        if (kp > qp || qp >= len || kp >= len) s = -INFINITY;
      }
      if (pm >= 0 && static_cast<const uint8_t *>(a.mask)[pm * sbs * sbs + idx] != 0) s = -INFINITY;
      t.s[i * ld + j] = s;
    }
  }
  __syncthreads();
}

template <typename Tr>
__global__ __launch_bounds__(kThreads) void attn_fwd_generic_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  extern __shared__ float smem[];
  const int sbs = a.sbs;
  const int ld = sbs + 1;
  Tiles t{smem, smem + sbs * ld, smem + 2 * sbs * ld};
  float *row_m = smem + 3 * sbs * ld;
  float *row_l = row_m + sbs;
  float *row_alpha = row_l + sbs;

  const int64_t b = blockIdx.x / a.nq, qb = blockIdx.x % a.nq;
  const int64_t h = blockIdx.y;
  const int own = sbs * sbs / kThreads;
  const bool has_o = h < a.nhv;
  int64_t po = -1;
  if (has_o) {
    po = a.pidx_o[(b * a.nq + qb) * a.nhv + h];
    if (po >= a.n_o_blocks) po = -1;
  }
  // this workgroup has nothing to write (lse belongs to slice 0)
  if (po < 0 && h != 0) return;

  if (threadIdx.x < sbs) {
    row_m[threadIdx.x] = -INFINITY;
    row_l[threadIdx.x] = 0.f;
  }
  float o[kMaxOwn];
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) o[m] = 0.f;

  const int k_begin = a.key_offsets[b * a.nq + qb], k_end = a.key_offsets[b * a.nq + qb + 1];
  for (int e = k_begin; e < k_end; ++e) {
    const int64_t kb = a.key_indices[e];
    score_tile<Tr>(a, t, b, qb, kb);
    // online softmax, one thread per query row
    if (threadIdx.x < sbs) {
      const int i = threadIdx.x;
      float *srow = t.s + i * ld;
      const float m_old = row_m[i];
      float m_new = m_old;
      for (int j = 0; j < sbs; ++j) m_new = fmaxf(m_new, srow[j]);
      const bool both_ninf = (m_old == -INFINITY) && (m_new == -INFINITY);
      const float alpha = both_ninf ? 1.f : exp2f(m_old - m_new);
      float sum = 0.f;
      for (int j = 0; j < sbs; ++j) {
        const float s = srow[j];
        float p = exp2f(s - m_new);
        if (s == -INFINITY && m_new == -INFINITY) p = 0.f;
        sum += p;
        srow[j] = Tr::widen(Tr::round(p));
      }
      row_l[i] = row_l[i] * alpha + sum;
      row_m[i] = m_new;
      row_alpha[i] = alpha;
    }
    __syncthreads();
    if (po >= 0) {
      const int64_t pv = a.pidx_v[(b * a.nk + kb) * a.nhv + h];
      const bool has_v = pv >= 0 && pv < a.n_v_blocks;
      if (has_v) load_block<Tr>(t.a, static_cast<const E *>(a.v) + pv * sbs * sbs, sbs, false);
      __syncthreads();
#pragma unroll
      for (int m = 0; m < kMaxOwn; ++m) {
        if (m < own) {
          const int idx = threadIdx.x + kThreads * m;
          const int i = idx / sbs, c = idx % sbs;
          float v = o[m] * row_alpha[i];
          if (has_v) {
            float dot = 0.f;
            for (int j = 0; j < sbs; ++j) dot = fmaf(t.s[i * ld + j], t.a[j * ld + c], dot);
            v += dot;
          }
          o[m] = v;
        }
      }
    }
    __syncthreads();
  }
  __syncthreads();
  if (po >= 0) {
    E *ob = static_cast<E *>(a.o) + po * sbs * sbs;
#pragma unroll
    for (int m = 0; m < kMaxOwn; ++m) {
      if (m < own) {
        const int idx = threadIdx.x + kThreads * m;
        const int i = idx / sbs;
        const float l = row_l[i];
        ob[idx] = Tr::round(l != 0.f ? o[m] / l : 0.f);
      }
    }
  }
  if (h == 0 && threadIdx.x < sbs) {
    const float l = row_l[threadIdx.x];
    a.lse[(b * a.nq + qb) * sbs + threadIdx.x] = (l != 0.f) ? row_m[threadIdx.x] + log2f(l) : -INFINITY;
  }
}

// delta[b, qb, i] = sum over active output slices of rowsum(o * do)
template <typename Tr>
__global__ __launch_bounds__(64) void attn_delta_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  const int sbs = a.sbs;
  const int64_t row = blockIdx.x;  // b * nq + qb
  const int lane = threadIdx.x;
  // lanes_per_row lanes share one query row
  const int lpr = 64 / sbs > 0 ? 64 / sbs : 1;
  for (int i0 = 0; i0 < sbs; i0 += (64 / lpr)) {
    const int i = i0 + lane / lpr;
    float acc = 0.f;
    if (i < sbs) {
      for (int64_t h = 0; h < a.nhv; ++h) {
        const int64_t po = a.pidx_o[row * a.nhv + h];
        if (po < 0 || po >= a.n_o_blocks) continue;
        const E *ob = static_cast<const E *>(a.o) + po * sbs * sbs + i * sbs;
        const E *gb = static_cast<const E *>(a.d_o) + po * sbs * sbs + i * sbs;
        for (int c = lane % lpr; c < sbs; c += lpr) acc = fmaf(Tr::widen(ob[c]), Tr::widen(gb[c]), acc);
      }
    }
    for (int d = 1; d < lpr; d <<= 1) acc += __shfl_xor(acc, d);
    if (i < sbs && (lane % lpr) == 0) a.delta[row * sbs + i] = acc;
  }
}

// After score_tile: t.s <- p (fp32) for this pair and returns dp - delta per owned element in `dpd`.
template <typename Tr>
__device__ inline void prob_and_dp(const bsa_attn_args &a, const Tiles &t, int64_t b, int64_t qb, int64_t kb,
                                   float (&dpd)[kMaxOwn]) {
  using E = typename Tr::elem_t;
  const int sbs = a.sbs;
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
  const float *lse = a.lse + (b * a.nq + qb) * sbs;
  const float *delta = a.delta + (b * a.nq + qb) * sbs;
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      const int i = idx / sbs, j = idx % sbs;
      const float mrow = lse[i];
      const bool valid = mrow != -INFINITY;
      const float p = valid ? exp2f(t.s[i * ld + j] - mrow) : 0.f;
      t.s[i * ld + j] = p;
    }
  }
  float acc[kMaxOwn];
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) acc[m] = 0.f;
  for (int64_t h = 0; h < a.nhv; ++h) {
    const int64_t po = a.pidx_o[(b * a.nq + qb) * a.nhv + h];
    const int64_t pv = a.pidx_v[(b * a.nk + kb) * a.nhv + h];
    if (po < 0 || pv < 0 || po >= a.n_o_blocks || pv >= a.n_v_blocks) continue;
    __syncthreads();
    load_block<Tr>(t.a, static_cast<const E *>(a.d_o) + po * sbs * sbs, sbs, false);
    load_block<Tr>(t.b, static_cast<const E *>(a.v) + pv * sbs * sbs, sbs, true);
    __syncthreads();
    tile_mac(acc, t.a, t.b, sbs);
  }
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      dpd[m] = acc[m] - delta[idx / sbs];
    }
  }
  __syncthreads();
}

// out[m] += sum_i round(S[i][j]) * A[i][c] for owned (j, c)
template <typename Tr>
__device__ inline void tile_mac_t(float (&acc)[kMaxOwn], const float *S, const float *A, int sbs, float factor) {
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      const int j = idx / sbs, c = idx % sbs;
      float dot = 0.f;
      for (int i = 0; i < sbs; ++i) dot = fmaf(Tr::widen(Tr::round(S[i * ld + j])), A[i * ld + c], dot);
      acc[m] += dot * factor;
    }
  }
}

// grid (B * nk, max(nh, nhv)): dK slice h and dV slice h of one key block, plus dBias from slice 0
template <typename Tr>
__global__ __launch_bounds__(kThreads) void attn_dkdv_generic_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  extern __shared__ float smem[];
  const int sbs = a.sbs;
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
  Tiles t{smem, smem + sbs * ld, smem + 2 * sbs * ld};
  const int64_t b = blockIdx.x / a.nk, kb = blockIdx.x % a.nk;
  const int64_t h = blockIdx.y;
  int64_t pk = -1, pv = -1;
  if (h < a.nh) pk = a.pidx_k[(b * a.nk + kb) * a.nh + h];
  if (h < a.nhv) pv = a.pidx_v[(b * a.nk + kb) * a.nhv + h];
  if (pk >= a.n_k_blocks) pk = -1;
  if (pv >= a.n_v_blocks) pv = -1;
  const bool want_dbias = (h == 0) && a.dbias != nullptr;
  if (pk < 0 && pv < 0 && !want_dbias) return;

  float dk[kMaxOwn], dv[kMaxOwn];
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) dk[m] = dv[m] = 0.f;

  const int q_begin = a.query_offsets[b * a.nk + kb], q_end = a.query_offsets[b * a.nk + kb + 1];
  for (int e = q_begin; e < q_end; ++e) {
    const int64_t qb = a.query_indices[e];
    score_tile<Tr>(a, t, b, qb, kb);
    float dpd[kMaxOwn];
    prob_and_dp<Tr>(a, t, b, qb, kb, dpd);
    // dV += round(p)^T dO_h
    if (pv >= 0) {
      const int64_t po = a.pidx_o[(b * a.nq + qb) * a.nhv + h];
      if (po >= 0 && po < a.n_o_blocks) {
        load_block<Tr>(t.a, static_cast<const E *>(a.d_o) + po * sbs * sbs, sbs, false);
        __syncthreads();
        tile_mac_t<Tr>(dv, t.s, t.a, sbs, 1.f);
      }
    }
    __syncthreads();
    // p -> ds in place (each thread rewrites the elements it owns)
    int64_t pb = -1;
    if (want_dbias) {
      pb = a.pidx_bias[(b * a.nq + qb) * a.nk + kb];
      if (pb >= a.n_bias_blocks) pb = -1;
    }
#pragma unroll
    for (int m = 0; m < kMaxOwn; ++m) {
      if (m < own) {
        const int idx = threadIdx.x + kThreads * m;
        const int i = idx / sbs, j = idx % sbs;
        const float ds = t.s[i * ld + j] * dpd[m];
        t.s[i * ld + j] = ds;
        // every (query block, key block) pair is visited once, so this is a plain store
        if (pb >= 0) a.dbias[pb * sbs * sbs + idx] = ds;
      }
    }
    __syncthreads();
    // dK += round(ds)^T Q_h * scale
    if (pk >= 0) {
      const int64_t pq = a.pidx_q[(b * a.nq + qb) * a.nh + h];
      if (pq >= 0 && pq < a.n_q_blocks) {
        load_block<Tr>(t.a, static_cast<const E *>(a.q) + pq * sbs * sbs, sbs, false);
        __syncthreads();
        tile_mac_t<Tr>(dk, t.s, t.a, sbs, a.scale);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      if (pk >= 0) static_cast<E *>(a.dk)[pk * sbs * sbs + idx] = Tr::round(dk[m]);
      if (pv >= 0) static_cast<E *>(a.dv)[pv * sbs * sbs + idx] = Tr::round(dv[m]);
    }
  }
}

// grid (B * nq, nh): dQ slice h of one query block
template <typename Tr>
__global__ __launch_bounds__(kThreads) void attn_dq_generic_kernel(bsa_attn_args a) {
  using E = typename Tr::elem_t;
  extern __shared__ float smem[];
  const int sbs = a.sbs;
  const int ld = sbs + 1;
  const int own = sbs * sbs / kThreads;
  Tiles t{smem, smem + sbs * ld, smem + 2 * sbs * ld};
  const int64_t b = blockIdx.x / a.nq, qb = blockIdx.x % a.nq;
  const int64_t h = blockIdx.y;
  int64_t pq = a.pidx_q[(b * a.nq + qb) * a.nh + h];
  if (pq < 0 || pq >= a.n_q_blocks) return;

  float dq[kMaxOwn];
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) dq[m] = 0.f;

  const int k_begin = a.key_offsets[b * a.nq + qb], k_end = a.key_offsets[b * a.nq + qb + 1];
  for (int e = k_begin; e < k_end; ++e) {
    const int64_t kb = a.key_indices[e];
    score_tile<Tr>(a, t, b, qb, kb);
    float dpd[kMaxOwn];
    prob_and_dp<Tr>(a, t, b, qb, kb, dpd);
#pragma unroll
    for (int m = 0; m < kMaxOwn; ++m) {
      if (m < own) {
        const int idx = threadIdx.x + kThreads * m;
        const int i = idx / sbs, j = idx % sbs;
        t.s[i * ld + j] = Tr::widen(Tr::round(t.s[i * ld + j] * dpd[m]));
      }
    }
    const int64_t pk = a.pidx_k[(b * a.nk + kb) * a.nh + h];
    if (pk >= 0 && pk < a.n_k_blocks) {
      load_block<Tr>(t.a, static_cast<const E *>(a.k) + pk * sbs * sbs, sbs, false);
      __syncthreads();
      // dQ[i][c] += sum_j ds[i][j] K[j][c] * scale
#pragma unroll
      for (int m = 0; m < kMaxOwn; ++m) {
        if (m < own) {
          const int idx = threadIdx.x + kThreads * m;
          const int i = idx / sbs, c = idx % sbs;
          float dot = 0.f;
          for (int j = 0; j < sbs; ++j) dot = fmaf(t.s[i * ld + j], t.a[j * ld + c], dot);
          dq[m] += dot * a.scale;
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int m = 0; m < kMaxOwn; ++m) {
    if (m < own) {
      const int idx = threadIdx.x + kThreads * m;
      static_cast<E *>(a.dq)[pq * sbs * sbs + idx] = Tr::round(dq[m]);
    }
  }
}

template <typename E>
__global__ void fill_zero_kernel(E *p, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = (E)0;
}

template <typename E>
int zero(E *p, int64_t n, hipStream_t s) {
  if (!p || n <= 0) return BSA_OK;
  int64_t blocks = cdiv(n, 256);
  if (blocks > 65536) blocks = 65536;
  fill_zero_kernel<E><<<(unsigned)blocks, 256, 0, s>>>(p, n);
  return check_launch("fill_zero_kernel");
}

size_t tile_lds_bytes(int sbs) { return (size_t)(3 * sbs * (sbs + 1) + 3 * sbs) * sizeof(float); }

template <typename Tr>
int fwd_impl(const bsa_attn_args &a, hipStream_t s) {
  const int64_t rows = a.B * a.nq;
  if (rows == 0) return BSA_OK;
  dim3 grid((unsigned)rows, (unsigned)(a.nhv > 0 ? a.nhv : 1));
  attn_fwd_generic_kernel<Tr><<<grid, kThreads, tile_lds_bytes(a.sbs), s>>>(a);
  return check_launch("attn_fwd_generic_kernel");
}

template <typename Tr>
int bwd_impl(const bsa_attn_args &a, hipStream_t s) {
  using E = typename Tr::elem_t;
  const int64_t bs = (int64_t)a.sbs * a.sbs;
  // blocks no workgroup reaches (inactive counterpart slices) and bias blocks outside the attention layout stay zero
  if (int rc = zero(static_cast<E *>(a.dq), a.n_q_blocks * bs, s)) return rc;
  if (int rc = zero(static_cast<E *>(a.dk), a.n_k_blocks * bs, s)) return rc;
  if (int rc = zero(static_cast<E *>(a.dv), a.n_v_blocks * bs, s)) return rc;
  if (int rc = zero(a.dbias, a.n_bias_blocks * bs, s)) return rc;
  const int64_t qrows = a.B * a.nq, krows = a.B * a.nk;
  if (qrows > 0) {
    attn_delta_kernel<Tr><<<(unsigned)qrows, 64, 0, s>>>(a);
    if (int rc = check_launch("attn_delta_kernel")) return rc;
  }
  const int64_t slices = a.nh > a.nhv ? a.nh : a.nhv;
  if (krows > 0 && slices > 0) {
    dim3 grid((unsigned)krows, (unsigned)slices);
    attn_dkdv_generic_kernel<Tr><<<grid, kThreads, tile_lds_bytes(a.sbs), s>>>(a);
    if (int rc = check_launch("attn_dkdv_generic_kernel")) return rc;
  } else if (krows > 0 && a.dbias) {
    dim3 grid((unsigned)krows, 1);
    attn_dkdv_generic_kernel<Tr><<<grid, kThreads, tile_lds_bytes(a.sbs), s>>>(a);
    if (int rc = check_launch("attn_dkdv_generic_kernel")) return rc;
  }
  if (qrows > 0 && a.nh > 0) {
    dim3 grid((unsigned)qrows, (unsigned)a.nh);
    attn_dq_generic_kernel<Tr><<<grid, kThreads, tile_lds_bytes(a.sbs), s>>>(a);
    if (int rc = check_launch("attn_dq_generic_kernel")) return rc;
  }
  return BSA_OK;
}

}  // namespace

int attn_fwd_generic(const bsa_attn_args &a, hipStream_t s) {
  switch (a.dtype) {
    case BSA_BF16: return fwd_impl<AttnBf16>(a, s);
    case BSA_F16: return fwd_impl<AttnF16>(a, s);
    default: return fwd_impl<AttnF32>(a, s);
  }
}

int attn_bwd_generic(const bsa_attn_args &a, hipStream_t s) {
  switch (a.dtype) {
    case BSA_BF16: return bwd_impl<AttnBf16>(a, s);
    case BSA_F16: return bwd_impl<AttnF16>(a, s);
    default: return bwd_impl<AttnF32>(a, s);
  }
}

}  // namespace bsa
