// Gather of head / relation rows fused with the model interaction -> one query vector per pair.
// One wavefront per (head, relation) pair; both rows are staged in LDS as fp32, normalised
// there if requested, and combined into Q[b, :] (and the per-row scalar bias of Keci).
//
// Head direction (pairs are (relation, tail), the unknown is the head): every model's triple score
// is linear in the head row, score(x, r, t) = Q'(r, t) . E[x].  DistMult: r * t.  ComplEx:
// conj(r) * t as complex numbers.  QMult: t (x) conj(r^) as quaternions.  Keci: the coefficient of
// each head component, including those of the sigma sums (which hold h and r but not t).  OMult:
// the coefficient of head part i is sum_j sign[j][i] * r^_(i xor j) * t_j.
#include "kge_internal.h"

namespace kge {
namespace {

struct QueryArgs {
  const void* ent;
  const float* ent_scale;
  const void* rel;
  const float* coeff_p;
  const float* coeff_q;
  const float* coeff_r;
  const int64_t* hr;
  float* Q;
  float* bias;
  kge_norm_params norm;
  kge_dropout_params drop;  // all masks null: no dropout
  int64_t B, N, R;
  int d, p, q, r, normalize_relation;
  int head_mode;  // pairs are (relation, tail) and Q is the head-direction query
};

// torch.nn.Dropout in training mode as a factor: 1 / (1 - rate) for a kept element, 0 for a dropped one (1 without a mask)
__device__ __forceinline__ float drop_factor(const uint8_t* keep, int64_t idx, float scale) {
  return keep ? (keep[idx] ? scale : 0.f) : 1.f;
}

template <int DT>
__device__ __forceinline__ float load_elem(const void* base, int64_t row, int d, int k, const float* scale) {
  if (DT == KGE_F32) return ((const float*)base)[row * d + k];
  if (DT == KGE_BF16) {
    uint32_t u = ((const uint16_t*)base)[row * d + k];
    return __uint_as_float(u << 16);
  }
  return (float)((const int8_t*)base)[row * d + k] * scale[row];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ void normalise_row(float* x, int d, int lane, int kind, float eps, const float* a, const float* b) {
  if (kind == KGE_NORM_LAYERNORM) {
    float s = 0.f;
    for (int k = lane; k < d; k += 64) s += x[k];
    float mu = wave_sum(s) / (float)d;
    float v = 0.f;
    for (int k = lane; k < d; k += 64) {
      float t = x[k] - mu;
      v += t * t;
    }
    float var = wave_sum(v) / (float)d;
    float inv = 1.0f / sqrtf(var + eps);
    for (int k = lane; k < d; k += 64) x[k] = (x[k] - mu) * inv * a[k] + b[k];
  } else if (kind == KGE_NORM_BATCHNORM1D) {
    for (int k = lane; k < d; k += 64) x[k] = (x[k] - a[k]) / sqrtf(b[k] + eps);
  }
}

template <int EDT, int RDT>
__global__ void __launch_bounds__(64) build_query_kernel(QueryArgs a, int model) {
  extern __shared__ float lds[];
  const int d = a.d;
  float* sh = lds;
  float* sr = lds + d;
  const int lane = threadIdx.x;
  const int64_t b = blockIdx.x;
  // the entity row of the pair (head, or tail in head mode) goes to sh, the relation row to sr
  const int64_t h_id = a.hr[2 * b + (a.head_mode ? 1 : 0)], r_id = a.hr[2 * b + (a.head_mode ? 0 : 1)];
  float* q = a.Q + b * d;
  if (h_id < 0 || h_id >= a.N || r_id < 0 || r_id >= a.R) {
    const float nan = __uint_as_float(0x7fc00000u);
    for (int k = lane; k < d; k += 64) q[k] = nan;
    if (lane == 0) a.bias[b] = nan;
    return;
  }
  for (int k = lane; k < d; k += 64) {
    sh[k] = load_elem<EDT>(a.ent, h_id, d, k, a.ent_scale) * drop_factor(a.drop.keep_h, b * d + k, a.drop.scale_in);
    sr[k] = load_elem<RDT>(a.rel, r_id, d, k, nullptr) * drop_factor(a.drop.keep_r, b * d + k, a.drop.scale_in);
  }
  __syncthreads();
  if (a.norm.kind != KGE_NORM_NONE) {
    normalise_row(sh, d, lane, a.norm.kind, a.norm.eps, a.norm.h_a, a.norm.h_b);
    normalise_row(sr, d, lane, a.norm.kind, a.norm.eps, a.norm.r_a, a.norm.r_b);
    __syncthreads();
  }
  float bias = 0.f;
  if (model == KGE_DISTMULT) {
    for (int k = lane; k < d; k += 64)
      q[k] = (sh[k] * sr[k]) * drop_factor(a.drop.keep_q, b * d + k, a.drop.scale_hidden);
  } else if (model == KGE_COMPLEX) {
    const int d2 = d >> 1;
    const float conj = a.head_mode ? -1.f : 1.f;
    for (int k = lane; k < d2; k += 64) {
      float hr_ = sh[k], hi_ = sh[k + d2], rr_ = sr[k], ri_ = conj * sr[k + d2];
      q[k] = hr_ * rr_ - hi_ * ri_;
      q[k + d2] = hr_ * ri_ + hi_ * rr_;
    }
  } else if (model == KGE_QMULT) {
    if (a.normalize_relation) {
      // groups of 4 consecutive elements, x / max(||x||, 1e-12)
      for (int g = lane; g < (d >> 2); g += 64) {
        float x0 = sr[4 * g], x1 = sr[4 * g + 1], x2 = sr[4 * g + 2], x3 = sr[4 * g + 3];
        float n = sqrtf(x0 * x0 + x1 * x1 + x2 * x2 + x3 * x3);
        float den = fmaxf(n, 1e-12f);
        sr[4 * g] = x0 / den;
        sr[4 * g + 1] = x1 / den;
        sr[4 * g + 2] = x2 / den;
        sr[4 * g + 3] = x3 / den;
      }
      __syncthreads();
    }
    const int d4 = d >> 2;
    const float conj = a.head_mode ? -1.f : 1.f;
    for (int g = lane; g < d4; g += 64) {
      float ah = sh[g], bh = sh[g + d4], ch = sh[g + 2 * d4], dh = sh[g + 3 * d4];
      float ar = sr[g], br = conj * sr[g + d4], cr = conj * sr[g + 2 * d4], dr = conj * sr[g + 3 * d4];
      q[g] = ah * ar - bh * br - ch * cr - dh * dr;
      q[g + d4] = ah * br + bh * ar + ch * dr - dh * cr;
      q[g + 2 * d4] = ah * cr - bh * dr + ch * ar + dh * br;
      q[g + 3 * d4] = ah * dr + bh * cr - ch * br + dh * ar;
    }
  } else if (model == KGE_OMULT) {
    // octonion product e_j = sum_i sign[j][i] * x_i * y_(i xor j); bit i of OCT_MINUS[j] set = minus
    constexpr unsigned char OCT_MINUS[8] = {0xfe, 0x68, 0xc2, 0xa4, 0x0e, 0x54, 0x98, 0x32};
    const int d8 = d >> 3;
    for (int g = lane; g < d8; g += 64) {
      float x[8], y[8], o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        x[i] = sh[g + i * d8];
        y[i] = sr[g + i * d8];
      }
      if (a.normalize_relation) {  // no epsilon, as the reference: a zero octonion gives NaN
        float n2 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) n2 += y[i] * y[i];
        const float den = sqrtf(n2);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = y[i] / den;
      }
      if (!a.head_mode) {  // x = head: o_j = sum_i sign[j][i] x_i y_(i^j)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float acc = 0.f;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float t = x[i] * y[i ^ j];
            acc += ((OCT_MINUS[j] >> i) & 1) ? -t : t;
          }
          o[j] = acc;
        }
      } else {  // x = tail: coefficient of head part i: sum_j sign[j][i] y_(i^j) x_j
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float acc = 0.f;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float t = y[i ^ j] * x[j];
            acc += ((OCT_MINUS[j] >> i) & 1) ? -t : t;
          }
          o[i] = acc;
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) q[g + i * d8] = o[i];
    }
  } else if (a.head_mode) {  // KGE_KECI / KGE_DECAL, head direction: sh holds the tail row (its parts are not scaled)
    const int p = a.p, qn = a.q, kn = a.r;
    const int r = d / (p + qn + kn + 1);
    const int qoff = r + r * p, koff = qoff + r * qn;
    for (int k = lane; k < r * p; k += 64) sr[r + k] *= a.coeff_p[k % p];
    for (int k = lane; k < r * qn; k += 64) sr[qoff + k] *= a.coeff_q[k % qn];
    for (int k = lane; k < r * kn; k += 64) sr[koff + k] *= a.coeff_r[k % kn];
    __syncthreads();
    for (int rho = lane; rho < r; rho += 64) {
      const float t0 = sh[rho], r0 = sr[rho];
      const float* tp = sh + r + rho * p;
      const float* rp = sr + r + rho * p;
      const float* tq = sh + qoff + rho * qn;
      const float* rq = sr + qoff + rho * qn;
      const float* tk = sh + koff + rho * kn;
      const float* rk = sr + koff + rho * kn;
      float q0 = r0 * t0, sum_rp = 0.f, sum_rq = 0.f, sum_rk = 0.f;
      for (int i = 0; i < p; ++i) {
        q0 += rp[i] * tp[i];
        sum_rp += rp[i];
      }
      for (int j = 0; j < qn; ++j) {
        q0 += rq[j] * tq[j];
        sum_rq += rq[j];
      }
      for (int l = 0; l < kn; ++l) {
        q0 += rk[l] * tk[l];
        sum_rk += rk[l];
      }
      q[rho] = q0;
      const bool pq = p >= 2 && qn >= 2, pr = p >= 2 && kn >= 2, qr = qn >= 2 && kn >= 2;
      float before = 0.f;  // sum of rp[k], k < i
      for (int i = 0; i < p; ++i) {
        float v = rp[i] * t0 + r0 * tp[i];
        if (p >= 2) v += (sum_rp - before - rp[i]) - before;  // d sigma_pp / d hp_i
        if (pq) v += sum_rq;                                   // d sigma_pq / d hp_i
        if (pr) v += sum_rk;                                   // d sigma_pr / d hp_i
        q[r + rho * p + i] = v * a.coeff_p[i];                 // the head's own part is scaled too
        before += rp[i];
      }
      before = 0.f;
      for (int j = 0; j < qn; ++j) {
        float v = -rq[j] * t0 + r0 * tq[j];
        if (qn >= 2) v += (sum_rq - before - rq[j]) - before;  // d sigma_qq / d hq_j
        if (pq) v -= sum_rp;                                   // d sigma_pq / d hq_j
        if (qr) v += sum_rk;                                   // d sigma_qr / d hq_j
        q[qoff + rho * qn + j] = v * a.coeff_q[j];
        before += rq[j];
      }
      before = 0.f;
      for (int l = 0; l < kn; ++l) {
        float v = r0 * tk[l];                                  // a degenerate base squares to zero: no t0 term
        if (kn >= 2) v += (sum_rk - before - rk[l]) - before;  // d sigma_rr / d hk_l
        if (pr) v -= sum_rp;                                   // d sigma_pr / d hk_l
        if (qr) v -= sum_rq;                                   // d sigma_qr / d hk_l
        q[koff + rho * kn + l] = v * a.coeff_r[l];
        before += rk[l];
      }
    }
  } else {  // KGE_KECI (r = 0) / KGE_DECAL
    const int p = a.p, qn = a.q, kn = a.r;
    const int r = d / (p + qn + kn + 1);
    // scale the p / q / r parts of both rows by their coefficients first, as the reference does
    for (int k = lane; k < r * p; k += 64) {
      float c = a.coeff_p[k % p];
      sh[r + k] *= c;
      sr[r + k] *= c;
    }
    const int qoff = r + r * p, koff = qoff + r * qn;
    for (int k = lane; k < r * qn; k += 64) {
      float c = a.coeff_q[k % qn];
      sh[qoff + k] *= c;
      sr[qoff + k] *= c;
    }
    for (int k = lane; k < r * kn; k += 64) {
      float c = a.coeff_r[k % kn];
      sh[koff + k] *= c;
      sr[koff + k] *= c;
    }
    __syncthreads();
    for (int rho = lane; rho < r; rho += 64) {
      const float h0 = sh[rho], r0 = sr[rho];
      const float* hp = sh + r + rho * p;
      const float* rp = sr + r + rho * p;
      const float* hq = sh + qoff + rho * qn;
      const float* rq = sr + qoff + rho * qn;
      const float* hk = sh + koff + rho * kn;
      const float* rk = sr + koff + rho * kn;
      float q0 = h0 * r0;
      for (int i = 0; i < p; ++i) {
        q0 += hp[i] * rp[i];
        q[r + rho * p + i] = h0 * rp[i] + hp[i] * r0;
      }
      for (int j = 0; j < qn; ++j) {
        q0 -= hq[j] * rq[j];
        q[qoff + rho * qn + j] = h0 * rq[j] + hq[j] * r0;
      }
      for (int l = 0; l < kn; ++l) q[koff + rho * kn + l] = h0 * rk[l] + hk[l] * r0;
      q[rho] = q0;
      if (p >= 2)
        for (int i = 0; i < p - 1; ++i)
          for (int k = i + 1; k < p; ++k) bias += hp[i] * rp[k] - hp[k] * rp[i];
      if (qn >= 2)
        for (int j = 0; j < qn - 1; ++j)
          for (int k = j + 1; k < qn; ++k) bias += hq[j] * rq[k] - hq[k] * rq[j];
      if (kn >= 2)
        for (int l = 0; l < kn - 1; ++l)
          for (int k = l + 1; k < kn; ++k) bias += hk[l] * rk[k] - hk[k] * rk[l];
      if (p >= 2 && qn >= 2)
        for (int i = 0; i < p; ++i)
          for (int j = 0; j < qn; ++j) bias += hp[i] * rq[j] - hq[j] * rp[i];
      if (p >= 2 && kn >= 2)
        for (int i = 0; i < p; ++i)
          for (int l = 0; l < kn; ++l) bias += hp[i] * rk[l] - hk[l] * rp[i];
      if (qn >= 2 && kn >= 2)
        for (int j = 0; j < qn; ++j)
          for (int l = 0; l < kn; ++l) bias += hq[j] * rk[l] - hk[l] * rq[j];
    }
    bias = wave_sum(bias);
  }
  if (lane == 0) a.bias[b] = bias;
}

// ---- backward of the query builder ---------------------------------------------------------------
// Given dL/dQ[b, :] and dL/dbias[b], add dL/d(head row) to d_ent[h], dL/d(relation row) to d_rel[r] and, for
// the Clifford models, dL/d(coefficients) to d_coeff_*.  One wavefront per pair; rows that several pairs share
// are combined with floating-point atomics.  fp32 tables.
// NORM: the rows pass through LayerNorm / BatchNorm1d (running statistics) before the interaction, as in the forward:
// the interaction's gradients at the normalised rows are collected in LDS (every element is produced exactly once per
// pair) and sent through the normaliser's own backward before they are added to the tables; LayerNorm's weight and
// bias receive their gradients too.
struct QueryBwdArgs {
  const float* ent;
  const float* rel;
  const float* coeff_p;
  const float* coeff_q;
  const float* coeff_r;
  const int64_t* hr;
  const float* dQ;
  const float* dbias;
  float* d_ent;
  float* d_rel;
  float* d_coeff_p;
  float* d_coeff_q;
  float* d_coeff_r;
  int64_t B, N, R;
  int d, p, q, r, normalize_relation;
  kge_norm_params norm;
  float* dn_h_a;  // LayerNorm: gradient of the head normaliser's weight / bias, of the relation normaliser's (may be null)
  float* dn_h_b;
  float* dn_r_a;
  float* dn_r_b;
  // BatchNorm1d with the statistics of the batch (training mode): the gradients at the normalised rows are written
  // here, [B, d] each, for the passes that need sums over the batch (null: every other mode)
  float* dy_h;
  float* dy_r;
  kge_dropout_params drop;  // the masks of the forward (all null: none)
};

// One row through the backward of its normaliser: x the row the normaliser saw (after dropout, if any), dy the gradient
// at the normalised row (both in LDS); adds the gradient at the raw row to out[] (through the row's dropout mask
// `keep`, null: none) and LayerNorm's parameter gradients to dw[] / db[].
__device__ void normalise_row_backward(const float* x, const float* dy, int d, int lane, int kind, float eps,
                                       const float* a, const float* b, float* out, float* dw, float* db,
                                       const uint8_t* keep, float keep_scale) {
  if (kind == KGE_NORM_LAYERNORM) {
    // the statistics exactly as normalise_row forms them
    float s = 0.f;
    for (int k = lane; k < d; k += 64) s += x[k];
    const float mu = wave_sum(s) / (float)d;
    float v = 0.f;
    for (int k = lane; k < d; k += 64) {
      const float t = x[k] - mu;
      v += t * t;
    }
    const float var = wave_sum(v) / (float)d;
    const float inv = 1.0f / sqrtf(var + eps);
    // y = xh * w + b with xh = (x - mu) * inv:  dx = inv * (g - mean(g) - xh * mean(g * xh)),  g = dy * w
    float s1 = 0.f, s2 = 0.f;
    for (int k = lane; k < d; k += 64) {
      const float g = dy[k] * a[k];
      s1 += g;
      s2 += g * ((x[k] - mu) * inv);
    }
    const float m1 = wave_sum(s1) / (float)d, m2 = wave_sum(s2) / (float)d;
    for (int k = lane; k < d; k += 64) {
      const float xh = (x[k] - mu) * inv, g = dy[k] * a[k];
      atomicAdd(&out[k], inv * (g - m1 - xh * m2) * drop_factor(keep, k, keep_scale));
      if (dw) atomicAdd(&dw[k], dy[k] * xh);
      if (db) atomicAdd(&db[k], dy[k]);
    }
  } else {  // BatchNorm1d with running statistics: an elementwise affine map
    for (int k = lane; k < d; k += 64) atomicAdd(&out[k], dy[k] / sqrtf(b[k] + eps) * drop_factor(keep, k, keep_scale));
  }
}

template <bool NORM>
__global__ void __launch_bounds__(64) build_query_backward_kernel(QueryBwdArgs a, int model) {
  extern __shared__ float lds[];
  const int d = a.d;
  float* sh = lds;          // head row
  float* sr = lds + d;      // relation row
  float* sg = lds + 2 * d;  // dL/dQ row
  float* sdh = lds + 3 * d;  // NORM: gradient at the normalised head row, at the normalised relation row, and the
  float* sdr = lds + 4 * d;  // norms of the relation's quaternions before QMult's own normaliser
  float* sn = lds + 5 * d;
  const int lane = threadIdx.x;
  const int64_t b = blockIdx.x;
  const int64_t h_id = a.hr[2 * b], r_id = a.hr[2 * b + 1];
  if (h_id < 0 || h_id >= a.N || r_id < 0 || r_id >= a.R) {  // the forward gave NaN for this pair
    if constexpr (NORM) {
      if (a.dy_h) {
        for (int k = lane; k < d; k += 64) a.dy_h[b * d + k] = a.dy_r[b * d + k] = 0.f;
      }
    }
    return;
  }
  for (int k = lane; k < d; k += 64) {
    sh[k] = a.ent[h_id * d + k] * drop_factor(a.drop.keep_h, b * d + k, a.drop.scale_in);
    sr[k] = a.rel[r_id * d + k] * drop_factor(a.drop.keep_r, b * d + k, a.drop.scale_in);
    sg[k] = a.dQ[b * d + k] * drop_factor(a.drop.keep_q, b * d + k, a.drop.scale_hidden);
  }
  __syncthreads();
  if constexpr (NORM) {
    normalise_row(sh, d, lane, a.norm.kind, a.norm.eps, a.norm.h_a, a.norm.h_b);
    normalise_row(sr, d, lane, a.norm.kind, a.norm.eps, a.norm.r_a, a.norm.r_b);
    __syncthreads();
  }
  float* gh = a.d_ent + h_id * d;
  float* gr = a.d_rel + r_id * d;
  auto emit_h = [&](int k, float v) {
    if constexpr (NORM) sdh[k] = v;
    else atomicAdd(&gh[k], v * drop_factor(a.drop.keep_h, b * d + k, a.drop.scale_in));
  };
  auto emit_r = [&](int k, float v) {
    if constexpr (NORM) sdr[k] = v;
    else atomicAdd(&gr[k], v * drop_factor(a.drop.keep_r, b * d + k, a.drop.scale_in));
  };
  if (model == KGE_DISTMULT) {
    for (int k = lane; k < d; k += 64) {
      emit_h(k, sg[k] * sr[k]);
      emit_r(k, sg[k] * sh[k]);
    }
  } else if (model == KGE_COMPLEX) {
    const int d2 = d >> 1;
    for (int k = lane; k < d2; k += 64) {
      const float hr_ = sh[k], hi_ = sh[k + d2], rr_ = sr[k], ri_ = sr[k + d2], g0 = sg[k], g1 = sg[k + d2];
      emit_h(k, g0 * rr_ + g1 * ri_);
      emit_h(k + d2, -g0 * ri_ + g1 * rr_);
      emit_r(k, g0 * hr_ + g1 * hi_);
      emit_r(k + d2, -g0 * hi_ + g1 * hr_);
    }
  } else if (model == KGE_QMULT) {
    const int d4 = d >> 2;
    // sr <- normalised relation (groups of 4 consecutive elements)
    if (a.normalize_relation) {
      for (int g = lane; g < d4; g += 64) {
        const float x0 = sr[4 * g], x1 = sr[4 * g + 1], x2 = sr[4 * g + 2], x3 = sr[4 * g + 3];
        const float nrm = sqrtf(x0 * x0 + x1 * x1 + x2 * x2 + x3 * x3);
        if constexpr (NORM) sn[g] = nrm;
        const float den = fmaxf(nrm, 1e-12f);
        sr[4 * g] = x0 / den;
        sr[4 * g + 1] = x1 / den;
        sr[4 * g + 2] = x2 / den;
        sr[4 * g + 3] = x3 / den;
      }
      __syncthreads();
    }
    // gradient at the head parts and at the NORMALISED relation parts (block layout); the latter overwrite sh
    for (int g = lane; g < d4; g += 64) {
      const float ah = sh[g], bh = sh[g + d4], ch = sh[g + 2 * d4], dh = sh[g + 3 * d4];
      const float pr = sr[g], qr = sr[g + d4], ur = sr[g + 2 * d4], vr = sr[g + 3 * d4];
      const float G0 = sg[g], G1 = sg[g + d4], G2 = sg[g + 2 * d4], G3 = sg[g + 3 * d4];
      emit_h(g, G0 * pr + G1 * qr + G2 * ur + G3 * vr);
      emit_h(g + d4, -G0 * qr + G1 * pr - G2 * vr + G3 * ur);
      emit_h(g + 2 * d4, -G0 * ur + G1 * vr + G2 * pr - G3 * qr);
      emit_h(g + 3 * d4, -G0 * vr - G1 * ur + G2 * qr + G3 * pr);
      sh[g] = G0 * ah + G1 * bh + G2 * ch + G3 * dh;
      sh[g + d4] = -G0 * bh + G1 * ah + G2 * dh - G3 * ch;
      sh[g + 2 * d4] = -G0 * ch - G1 * dh + G2 * ah + G3 * bh;
      sh[g + 3 * d4] = -G0 * dh + G1 * ch - G2 * bh + G3 * ah;
    }
    __syncthreads();
    if (!a.normalize_relation) {
      for (int k = lane; k < d; k += 64) emit_r(k, sh[k]);
    } else {
      // y = x / max(|x|, eps) per group of 4 consecutive elements: dx = (dy - y (y . dy)) / |x|, or dy / eps
      // where the norm was clamped
      for (int g = lane; g < d4; g += 64) {
        float n;
        if constexpr (NORM) {
          n = sn[g];
        } else {
          const float* raw = a.rel + r_id * d + 4 * g;
          const int64_t at = b * d + 4 * g;
          const float x0 = raw[0] * drop_factor(a.drop.keep_r, at, a.drop.scale_in);
          const float x1 = raw[1] * drop_factor(a.drop.keep_r, at + 1, a.drop.scale_in);
          const float x2 = raw[2] * drop_factor(a.drop.keep_r, at + 2, a.drop.scale_in);
          const float x3 = raw[3] * drop_factor(a.drop.keep_r, at + 3, a.drop.scale_in);
          n = sqrtf(x0 * x0 + x1 * x1 + x2 * x2 + x3 * x3);
        }
        const float y0 = sr[4 * g], y1 = sr[4 * g + 1], y2 = sr[4 * g + 2], y3 = sr[4 * g + 3];
        const float e0 = sh[4 * g], e1 = sh[4 * g + 1], e2 = sh[4 * g + 2], e3 = sh[4 * g + 3];
        if (n < 1e-12f) {
          emit_r(4 * g, e0 / 1e-12f);
          emit_r(4 * g + 1, e1 / 1e-12f);
          emit_r(4 * g + 2, e2 / 1e-12f);
          emit_r(4 * g + 3, e3 / 1e-12f);
        } else {
          const float dot = y0 * e0 + y1 * e1 + y2 * e2 + y3 * e3;
          emit_r(4 * g, (e0 - y0 * dot) / n);
          emit_r(4 * g + 1, (e1 - y1 * dot) / n);
          emit_r(4 * g + 2, (e2 - y2 * dot) / n);
          emit_r(4 * g + 3, (e3 - y3 * dot) / n);
        }
      }
    }
  } else if (model == KGE_OMULT) {
    constexpr unsigned char OCT_MINUS[8] = {0xfe, 0x68, 0xc2, 0xa4, 0x0e, 0x54, 0x98, 0x32};
    const int d8 = d >> 3;
    for (int g = lane; g < d8; g += 64) {
      float x[8], y[8], G[8], dx[8], dy[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        x[i] = sh[g + i * d8];
        y[i] = sr[g + i * d8];
        G[i] = sg[g + i * d8];
      }
      float den = 1.f;
      if (a.normalize_relation) {
        float n2 = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) n2 += y[i] * y[i];
        den = sqrtf(n2);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = y[i] / den;
      }
      // o_j = sum_i sign[j][i] x_i y_(i^j):  d x_i = sum_j sign[j][i] y_(i^j) G_j,  d y_m = sum_j sign[j][m^j] x_(m^j) G_j
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float ax = 0.f, ay = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float tx = y[i ^ j] * G[j];
          ax += ((OCT_MINUS[j] >> i) & 1) ? -tx : tx;
          const float ty = x[i ^ j] * G[j];
          ay += ((OCT_MINUS[j] >> (i ^ j)) & 1) ? -ty : ty;
        }
        dx[i] = ax;
        dy[i] = ay;
      }
      if (a.normalize_relation) {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) dot += y[i] * dy[i];
#pragma unroll
        for (int i = 0; i < 8; ++i) dy[i] = (dy[i] - y[i] * dot) / den;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        emit_h(g + i * d8, dx[i]);
        emit_r(g + i * d8, dy[i]);
      }
    }
  } else {  // KGE_KECI (r = 0) / KGE_DECAL
    const int p = a.p, qn = a.q, kn = a.r;
    const int re = d / (p + qn + kn + 1);
    const int poff = re, qoff = re + re * p, koff = qoff + re * qn;
    const float gb = a.dbias ? a.dbias[b] : 0.f;
    const bool pp = p >= 2, qq = qn >= 2, kk = kn >= 2;
    // coefficient of base i (p, then q, then r bases), the sign of its square, and its family
    auto coeff = [&](int i) { return i < p ? a.coeff_p[i] : i < p + qn ? a.coeff_q[i - p] : a.coeff_r[i - p - qn]; };
    auto col = [&](int rho, int i) {
      return i < p ? poff + rho * p + i : i < p + qn ? qoff + rho * qn + (i - p) : koff + rho * kn + (i - p - qn);
    };
    auto family = [&](int i) { return i < p ? 0 : i < p + qn ? 1 : 2; };
    const int nb = p + qn + kn;
    float dc[16];  // per-lane partial gradient of up to 16 coefficients (more are handled in further rounds)
    for (int i0 = 0; i0 < nb || i0 == 0; i0 += 16) {
#pragma unroll
      for (int u = 0; u < 16; ++u) dc[u] = 0.f;
      for (int rho = lane; rho < re; rho += 64) {
        const float h0 = sh[rho], r0 = sr[rho], G0 = sg[rho];
        // sums of the scaled parts of each family (for the sigma terms)
        float sum_h[3] = {0.f, 0.f, 0.f}, sum_r[3] = {0.f, 0.f, 0.f};
        float dh0 = G0 * r0, dr0 = G0 * h0;
        for (int i = 0; i < nb; ++i) {
          const float c = coeff(i), hs = c * sh[col(rho, i)], rs = c * sr[col(rho, i)], Gi = sg[col(rho, i)];
          sum_h[family(i)] += hs;
          sum_r[family(i)] += rs;
          dh0 += Gi * rs;
          dr0 += Gi * hs;
        }
        if (i0 == 0) {
          emit_h(rho, dh0);
          emit_r(rho, dr0);
        }
        const bool fam_on[3] = {pp, qq, kk};
        float before_h[3] = {0.f, 0.f, 0.f}, before_r[3] = {0.f, 0.f, 0.f};
        for (int i = 0; i < nb; ++i) {
          const int f = family(i);
          const float c = coeff(i), hraw = sh[col(rho, i)], rraw = sr[col(rho, i)], hs = c * hraw, rs = c * rraw;
          const float Gi = sg[col(rho, i)];
          const float sq = (f == 0) ? 1.f : (f == 1) ? -1.f : 0.f;  // e_i^2
          float dhs = sq * G0 * rs + Gi * r0;                       // gradient at the scaled head part
          float drs = sq * G0 * hs + Gi * h0;
          if (fam_on[f]) {  // same-family sigma: sum_{i<k} (h_i r_k - h_k r_i)
            dhs += gb * ((sum_r[f] - before_r[f] - rs) - before_r[f]);
            drs += gb * (before_h[f] - (sum_h[f] - before_h[f] - hs));
          }
          // cross-family sigmas (x, y) with x before y: sum (h_x r_y - h_y r_x), present when both counts >= 2
          for (int g2 = 0; g2 < 3; ++g2) {
            if (g2 == f || !fam_on[f] || !fam_on[g2]) continue;
            if (f < g2) {
              dhs += gb * sum_r[g2];
              drs -= gb * sum_h[g2];
            } else {
              dhs -= gb * sum_r[g2];
              drs += gb * sum_h[g2];
            }
          }
          before_h[f] += hs;
          before_r[f] += rs;
          if (i0 == 0) {
            emit_h(col(rho, i), c * dhs);
            emit_r(col(rho, i), c * drs);
          }
          if (i >= i0 && i < i0 + 16) dc[i - i0] += hraw * dhs + rraw * drs;
        }
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int i = i0 + u;
        if (i >= nb) break;  // uniform
        const float v = wave_sum(dc[u]);
        float* dst = i < p ? a.d_coeff_p : i < p + qn ? a.d_coeff_q : a.d_coeff_r;
        const int idx = i < p ? i : i < p + qn ? i - p : i - p - qn;
        if (lane == 0 && dst) atomicAdd(&dst[idx], v);
      }
    }
  }
  if constexpr (NORM) {
    // the raw rows once more, and each gradient through its normaliser
    __syncthreads();
    for (int k = lane; k < d; k += 64) {
      sh[k] = a.ent[h_id * d + k] * drop_factor(a.drop.keep_h, b * d + k, a.drop.scale_in);
      sr[k] = a.rel[r_id * d + k] * drop_factor(a.drop.keep_r, b * d + k, a.drop.scale_in);
    }
    __syncthreads();
    if (a.dy_h) {
      for (int k = lane; k < d; k += 64) {
        a.dy_h[b * d + k] = sdh[k];
        a.dy_r[b * d + k] = sdr[k];
      }
      return;
    }
    normalise_row_backward(sh, sdh, d, lane, a.norm.kind, a.norm.eps, a.norm.h_a, a.norm.h_b, gh, a.dn_h_a, a.dn_h_b,
                           a.drop.keep_h ? a.drop.keep_h + b * d : nullptr, a.drop.scale_in);
    normalise_row_backward(sr, sdr, d, lane, a.norm.kind, a.norm.eps, a.norm.r_a, a.norm.r_b, gr, a.dn_r_a, a.dn_r_b,
                           a.drop.keep_r ? a.drop.keep_r + b * d : nullptr, a.drop.scale_in);
  }
}

// ---- BatchNorm1d(affine=False) with the statistics of the batch (training mode) -------------------------------
// Sums over the batch per feature, for the head rows and the relation rows of the pairs: lanes along the features
// (whole lines per request), the four waves of a workgroup and the workgroups of grid.y along the batch, fp64
// partial sums met with atomics in sums[4][d].
//   GRAD == false: sum x, sum x^2 of the looked-up rows (-> mean and biased variance)
//   GRAD == true:  sum dy, sum dy * xh with xh = (x - mean) / sqrt(var + eps), dy read from dy_h / dy_r [B, d]
// A pair with an id outside its table poisons the sums with NaN (the forward gives NaN for it as well).
struct BnSumArgs {
  const float* ent;
  const float* rel;
  const int64_t* hr;
  const float* dy_h;
  const float* dy_r;
  kge_norm_params norm;
  kge_dropout_params drop;
  double* sums;
  int64_t B, N, R;
  int d;
};

template <bool GRAD>
__global__ void __launch_bounds__(256) bn_sums_kernel(BnSumArgs a) {
  __shared__ double part[4][4][64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int f = blockIdx.x * 64 + lane;
  const int d = a.d;
  const int64_t per = (a.B + gridDim.y - 1) / gridDim.y;
  const int64_t b0 = (int64_t)blockIdx.y * per, b1 = (b0 + per < a.B) ? b0 + per : a.B;
  double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
  float mh = 0.f, ih = 0.f, mr = 0.f, ir = 0.f;
  if (GRAD && f < d) {
    mh = a.norm.h_a[f];
    ih = 1.0f / sqrtf(a.norm.h_b[f] + a.norm.eps);
    mr = a.norm.r_a[f];
    ir = 1.0f / sqrtf(a.norm.r_b[f] + a.norm.eps);
  }
  for (int64_t b = b0 + w; b < b1; b += 4) {
    const int64_t h_id = a.hr[2 * b], r_id = a.hr[2 * b + 1];
    if (h_id < 0 || h_id >= a.N || r_id < 0 || r_id >= a.R) {
      s0 = s1 = s2 = s3 = __longlong_as_double(0x7ff8000000000000LL);
      continue;
    }
    if (f < d) {
      const float x = a.ent[h_id * d + f] * drop_factor(a.drop.keep_h, b * d + f, a.drop.scale_in);
      const float y = a.rel[r_id * d + f] * drop_factor(a.drop.keep_r, b * d + f, a.drop.scale_in);
      if (GRAD) {
        const float gh = a.dy_h[b * d + f], gr = a.dy_r[b * d + f];
        s0 += (double)gh;
        s1 += (double)gh * (double)((x - mh) * ih);
        s2 += (double)gr;
        s3 += (double)gr * (double)((y - mr) * ir);
      } else {
        s0 += (double)x;
        s1 += (double)x * (double)x;
        s2 += (double)y;
        s3 += (double)y * (double)y;
      }
    }
  }
  part[w][0][lane] = s0;
  part[w][1][lane] = s1;
  part[w][2][lane] = s2;
  part[w][3][lane] = s3;
  __syncthreads();
  if (f < d) {
    const double v = part[0][w][lane] + part[1][w][lane] + part[2][w][lane] + part[3][w][lane];  // wave w: sum w
    atomicAdd(&a.sums[(int64_t)w * d + f], v);
  }
}

__global__ void bn_zero_kernel(double* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.0;
}

// mean and biased variance of the batch, and the update of the running statistics torch.nn.BatchNorm1d makes in
// training mode: running = (1 - momentum) * running + momentum * (mean | variance * B / (B - 1))
__global__ void bn_finish_stats_kernel(const double* sums, int d, int64_t B, float momentum, float* h_mean, float* h_var,
                                       float* r_mean, float* r_var, float* run_h_mean, float* run_h_var,
                                       float* run_r_mean, float* run_r_var) {
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= d) return;
  const double n = (double)B, unb = n / (n - 1.0);
  for (int side = 0; side < 2; ++side) {
    const double mean = sums[(2 * side) * (int64_t)d + f] / n;
    double var = sums[(2 * side + 1) * (int64_t)d + f] / n - mean * mean;
    var = var < 0.0 ? 0.0 : var;  // (NaN stays NaN)
    (side ? r_mean : h_mean)[f] = (float)mean;
    (side ? r_var : h_var)[f] = (float)var;
    float* rm = side ? run_r_mean : run_h_mean;
    float* rv = side ? run_r_var : run_h_var;
    if (rm) rm[f] = (float)((1.0 - (double)momentum) * (double)rm[f] + (double)momentum * mean);
    if (rv) rv[f] = (float)((1.0 - (double)momentum) * (double)rv[f] + (double)momentum * var * unb);
  }
}

// dx = (dy - mean_B(dy) - xh * mean_B(dy * xh)) / sqrt(var + eps) per pair and feature, added to the tables' gradients
__global__ void __launch_bounds__(256) bn_backward_apply_kernel(BnSumArgs a, float* d_ent, float* d_rel) {
  const int d = a.d;
  const int f = blockIdx.x * 64 + (threadIdx.x & 63);
  if (f >= d) return;
  const double n = (double)a.B;
  const float mh = a.norm.h_a[f], ih = 1.0f / sqrtf(a.norm.h_b[f] + a.norm.eps);
  const float mr = a.norm.r_a[f], ir = 1.0f / sqrtf(a.norm.r_b[f] + a.norm.eps);
  const float h1 = (float)(a.sums[f] / n), h2 = (float)(a.sums[(int64_t)d + f] / n);
  const float r1 = (float)(a.sums[2 * (int64_t)d + f] / n), r2 = (float)(a.sums[3 * (int64_t)d + f] / n);
  for (int64_t b = (int64_t)blockIdx.y * 4 + (threadIdx.x >> 6); b < a.B; b += 4 * (int64_t)gridDim.y) {
    const int64_t h_id = a.hr[2 * b], r_id = a.hr[2 * b + 1];
    if (h_id < 0 || h_id >= a.N || r_id < 0 || r_id >= a.R) continue;
    const float kh = drop_factor(a.drop.keep_h, b * d + f, a.drop.scale_in);
    const float kr = drop_factor(a.drop.keep_r, b * d + f, a.drop.scale_in);
    const float xh = (a.ent[h_id * d + f] * kh - mh) * ih, yh = (a.rel[r_id * d + f] * kr - mr) * ir;
    atomicAdd(&d_ent[h_id * d + f], (a.dy_h[b * d + f] - h1 - xh * h2) * ih * kh);
    atomicAdd(&d_rel[r_id * d + f], (a.dy_r[b * d + f] - r1 - yh * r2) * ir * kr);
  }
}

// ---- the same for the models whose query vector is elementwise in part-strided positions ------------------------
// DistMult (1 part), ComplEx (2) and QMult (4), no normalisation layer: output element g of part j reads the head and
// relation rows at g + i * d / parts only, so one THREAD owns one g of one pair, loads its 2 x parts elements straight
// from the tables (lanes along g: whole lines per request), and stores its `parts` outputs; no LDS, no barrier, a
// handful of registers.  QMult's relation normaliser divides every 4 CONSECUTIVE elements by their norm
// (quaternion.py:28-43 on the flat row): the four lanes of a quad hold exactly such a group in every part (d / 4 is
// a multiple of 4 whenever it matters: otherwise the general kernel runs), so the norm is a quad reduction.
// A wave holds 64 x parts x 2 elements of reads in flight and nothing else, at full occupancy: the gather runs at
// the memory system's rate for small requests instead of one 512-byte pair per wave lifetime.
// VEC consecutive elements of a table row starting at element `off` (VEC = 4: one 16-, 8- or 4-byte load)
template <int DT, int VEC>
__device__ __forceinline__ void table_elems(const void* base, int64_t off, float (&v)[VEC]) {
  if (VEC == 4) {
    if (DT == KGE_F32) {
      const f32x4 x = *(const f32x4*)((const float*)base + off);
      v[0] = x[0]; v[1] = x[1]; v[2] = x[2]; v[3] = x[3];
    } else if (DT == KGE_BF16) {
      const u32x2 x = *(const u32x2*)((const uint16_t*)base + off);
      v[0] = __uint_as_float(x[0] << 16); v[1] = __uint_as_float(x[0] & 0xffff0000u);
      v[2] = __uint_as_float(x[1] << 16); v[3] = __uint_as_float(x[1] & 0xffff0000u);
    } else {
      const uint32_t x = *(const uint32_t*)((const int8_t*)base + off);
      v[0] = (float)(int8_t)x; v[1] = (float)(int8_t)(x >> 8); v[2] = (float)(int8_t)(x >> 16); v[3] = (float)(int8_t)(x >> 24);
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      if (DT == KGE_F32) v[i] = ((const float*)base)[off + i];
      else if (DT == KGE_BF16) v[i] = __uint_as_float((uint32_t)((const uint16_t*)base)[off + i] << 16);
      else v[i] = (float)((const int8_t*)base)[off + i];
    }
  }
}
// x0 + x1 + x2 + x3 over the four lanes of a quad, added in that order in every lane (the order of the general kernel)
__device__ __forceinline__ float quad_sum(float v, int lane) {
  const int q0 = lane & ~3;
  const float s0 = __shfl(v, q0, 64), s1 = __shfl(v, q0 + 1, 64), s2 = __shfl(v, q0 + 2, 64), s3 = __shfl(v, q0 + 3, 64);
  return s0 + s1 + s2 + s3;
}
// A thread owns VEC consecutive elements g .. g + VEC - 1 of every part (VEC = 4 when a part's length and the rows'
// addresses allow 16-byte accesses: one load per row and part, one 16-byte store per part, and the relation
// normaliser's group of four inside the thread; VEC = 1 otherwise).  A workgroup of 256 threads takes floor(256 / u)
// whole pairs when a part has at most 256 units (u = d / parts / VEC; `magic` = ceil(65536 / u) turns the thread number
// into (pair, unit) without a division), otherwise one 256-unit block of one pair (`blocks` blocks per pair).
template <int EDT, int RDT, int PARTS, int VEC>
__global__ void __launch_bounds__(256) build_query_flat_kernel(QueryArgs a, int units, int ppw, int magic, int blocks) {
  const int tid = threadIdx.x;
  const int dp = units * VEC;
  int64_t b;
  int u;
  bool live;
  if (blocks == 1) {
    const int pl = (tid * magic) >> 16;  // tid / units for tid < 256
    u = tid - pl * units;
    b = (int64_t)blockIdx.x * ppw + pl;
    live = pl < ppw && b < a.B;  // (lanes past the end stay in the quad reductions with zeros)
  } else {
    b = blockIdx.x / blocks;
    u = (int)(blockIdx.x - b * blocks) * 256 + tid;
    live = u < units;
    u = live ? u : 0;
  }
  const int g = u * VEC;
  int64_t e_id = 0, r_id = 0;
  if (live) {
    e_id = a.hr[2 * b + (a.head_mode ? 1 : 0)];
    r_id = a.hr[2 * b + (a.head_mode ? 0 : 1)];
  }
  const bool ok = live && e_id >= 0 && e_id < a.N && r_id >= 0 && r_id < a.R;
  float h[PARTS][VEC], r[PARTS][VEC];
#pragma unroll
  for (int j = 0; j < PARTS; ++j) {
    if (ok) {
      table_elems<EDT, VEC>(a.ent, e_id * a.d + g + j * dp, h[j]);
      table_elems<RDT, VEC>(a.rel, r_id * a.d + g + j * dp, r[j]);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) h[j][i] = r[j][i] = 0.f;
    }
  }
  if (EDT == KGE_I8) {
    const float sc = ok ? a.ent_scale[e_id] : 0.f;
#pragma unroll
    for (int j = 0; j < PARTS; ++j)
#pragma unroll
      for (int i = 0; i < VEC; ++i) h[j][i] *= sc;
  }
  if (PARTS == 4 && a.normalize_relation) {
    // every 4 consecutive elements of the flat relation row by their norm, x / max(||x||, 1e-12)
#pragma unroll
    for (int j = 0; j < PARTS; ++j) {
      float n;
      if (VEC == 4) n = sqrtf(r[j][0] * r[j][0] + r[j][1] * r[j][1] + r[j][2] * r[j][2] + r[j][3] * r[j][3]);
      else n = sqrtf(quad_sum(r[j][0] * r[j][0], tid & 63));
      const float den = fmaxf(n, 1e-12f);
#pragma unroll
      for (int i = 0; i < VEC; ++i) r[j][i] = r[j][i] / den;
    }
  }
  float o[PARTS][VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    if (PARTS == 1) {
      o[0][i] = h[0][i] * r[0][i];
    } else if (PARTS == 2) {
      const float ri = a.head_mode ? -r[1][i] : r[1][i];
      o[0][i] = h[0][i] * r[0][i] - h[1][i] * ri;
      o[1][i] = h[0][i] * ri + h[1][i] * r[0][i];
    } else {
      const float conj = a.head_mode ? -1.f : 1.f;
      const float ah = h[0][i], bh = h[1 % PARTS][i], ch = h[2 % PARTS][i], dh = h[3 % PARTS][i];
      const float ar = r[0][i], br = conj * r[1 % PARTS][i], cr = conj * r[2 % PARTS][i], dr = conj * r[3 % PARTS][i];
      o[0][i] = ah * ar - bh * br - ch * cr - dh * dr;
      o[1 % PARTS][i] = ah * br + bh * ar + ch * dr - dh * cr;
      o[2 % PARTS][i] = ah * cr - bh * dr + ch * ar + dh * br;
      o[3 % PARTS][i] = ah * dr + bh * cr - ch * br + dh * ar;
    }
  }
  if (!live) return;
  const float nan = __uint_as_float(0x7fc00000u);
  float* q = a.Q + b * a.d + g;
#pragma unroll
  for (int j = 0; j < PARTS; ++j) {
    if (VEC == 4) {
      f32x4 w = {ok ? o[j][0] : nan, ok ? o[j][1] : nan, ok ? o[j][2] : nan, ok ? o[j][3] : nan};
      *(f32x4*)(q + j * dp) = w;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) q[j * dp + i] = ok ? o[j][i] : nan;
    }
  }
  if (u == 0) a.bias[b] = ok ? 0.f : nan;
}

template <int EDT, int PARTS>
int launch_build_query_flat(const QueryArgs& a, int rel_dtype, hipStream_t st) {
  const int dp = a.d / PARTS;
  // 16-byte accesses: whole groups of four per part, rows that start on 16-byte (fp32), 8-byte (bf16), 4-byte (int8) bounds
  const int eb = EDT == KGE_F32 ? 4 : EDT == KGE_BF16 ? 2 : 1, rb = rel_dtype == KGE_F32 ? 4 : 2;
  const bool vec = dp % 4 == 0 && ((uintptr_t)a.ent % (4 * eb)) == 0 && ((uintptr_t)a.rel % (4 * rb)) == 0 &&
                   ((uintptr_t)a.Q % 16) == 0;
  const int units = vec ? dp / 4 : dp;
  const int ppw = units <= 256 ? 256 / units : 1, blocks = units <= 256 ? 1 : (units + 255) / 256;
  const int magic = (65536 + units - 1) / units;
  const int64_t nwg = blocks == 1 ? (a.B + ppw - 1) / ppw : a.B * blocks;
  KGE_REQUIRE(nwg <= 0x7fffffffLL, KGE_ERR_INVALID, "kge_build_query: B=%lld too large", (long long)a.B);
  const dim3 grid((unsigned)nwg), block(256);
  if (rel_dtype == KGE_F32) {
    if (vec) hipLaunchKernelGGL((build_query_flat_kernel<EDT, KGE_F32, PARTS, 4>), grid, block, 0, st, a, units, ppw, magic, blocks);
    else hipLaunchKernelGGL((build_query_flat_kernel<EDT, KGE_F32, PARTS, 1>), grid, block, 0, st, a, units, ppw, magic, blocks);
  } else {
    if (vec) hipLaunchKernelGGL((build_query_flat_kernel<EDT, KGE_BF16, PARTS, 4>), grid, block, 0, st, a, units, ppw, magic, blocks);
    else hipLaunchKernelGGL((build_query_flat_kernel<EDT, KGE_BF16, PARTS, 1>), grid, block, 0, st, a, units, ppw, magic, blocks);
  }
  KGE_LAUNCH_CHECK("build_query_flat_kernel");
  return KGE_OK;
}

template <int EDT>
int launch_build_query(const QueryArgs& a, int model, int rel_dtype, hipStream_t st) {
  const bool dropout = a.drop.keep_h || a.drop.keep_r || a.drop.keep_q;
  if (a.norm.kind == KGE_NORM_NONE && a.B > 0 && !dropout) {
    if (model == KGE_DISTMULT) return launch_build_query_flat<EDT, 1>(a, rel_dtype, st);
    if (model == KGE_COMPLEX) return launch_build_query_flat<EDT, 2>(a, rel_dtype, st);
    if (model == KGE_QMULT && (!a.normalize_relation || (a.d / 4) % 4 == 0)) return launch_build_query_flat<EDT, 4>(a, rel_dtype, st);
  }
  dim3 grid((unsigned)a.B), block(64);
  size_t shmem = 2 * (size_t)a.d * sizeof(float);
  if (rel_dtype == KGE_F32)
    hipLaunchKernelGGL((build_query_kernel<EDT, KGE_F32>), grid, block, shmem, st, a, model);
  else
    hipLaunchKernelGGL((build_query_kernel<EDT, KGE_BF16>), grid, block, shmem, st, a, model);
  KGE_LAUNCH_CHECK("build_query_kernel");
  return KGE_OK;
}

}  // namespace
}  // namespace kge

namespace kge {
namespace {
// keep_q is DistMult's dropout on h * r (dicee/models/real.py:32); no other model of this path has one
int check_dropout(const char* who, const kge_dropout_params* dp, int model) {
  KGE_REQUIRE(!dp->keep_q || model == KGE_DISTMULT, KGE_ERR_INVALID, "%s: keep_q is DistMult's hidden dropout only", who);
  KGE_REQUIRE(dp->scale_in >= 1.f && dp->scale_hidden >= 1.f && dp->scale_in < 1e30f && dp->scale_hidden < 1e30f,
              KGE_ERR_INVALID, "%s: scales must be 1 / (1 - rate) with a rate in [0, 1), got %g and %g", who,
              (double)dp->scale_in, (double)dp->scale_hidden);
  return KGE_OK;
}
}  // namespace
}  // namespace kge

static int build_query_impl(int head_mode, int model, int p, int q, int r, const void* ent, int ent_dtype,
                            const float* ent_scale, const void* rel, int rel_dtype, const float* coeff_p,
                            const float* coeff_q, const float* coeff_r, int normalize_relation, const kge_norm_params* norm,
                            const int64_t* hr, int64_t B, int64_t d, int64_t N, int64_t R, float* Q, float* bias,
                            void* stream, const kge_dropout_params* dropout = nullptr) {
  using namespace kge;
  clear_error();
  KGE_REQUIRE(!head_mode || !dropout, KGE_ERR_UNSUPPORTED, "kge_build_query_head: no dropout in the head direction");
  KGE_REQUIRE(!head_mode || !norm || norm->kind == KGE_NORM_NONE, KGE_ERR_UNSUPPORTED,
              "kge_build_query_head: a normalised head row is not a row of the table; only normalisation 'none'");
  KGE_REQUIRE(B >= 0 && N > 0 && R > 0, KGE_ERR_INVALID, "kge_build_query: B=%lld N=%lld R=%lld", (long long)B,
              (long long)N, (long long)R);
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(ent && rel && hr && Q && bias, KGE_ERR_INVALID, "kge_build_query: null pointer argument");
  KGE_REQUIRE(d >= 1 && d <= 8192, KGE_ERR_INVALID, "kge_build_query: d=%lld outside [1, 8192]", (long long)d);
  KGE_REQUIRE(B <= 0x7fffffff, KGE_ERR_INVALID, "kge_build_query: B=%lld too large", (long long)B);
  KGE_REQUIRE(ent_dtype == KGE_F32 || ent_dtype == KGE_BF16 || ent_dtype == KGE_I8, KGE_ERR_INVALID,
              "kge_build_query: unknown entity dtype %d", ent_dtype);
  KGE_REQUIRE(rel_dtype == KGE_F32 || rel_dtype == KGE_BF16, KGE_ERR_INVALID,
              "kge_build_query: relation dtype must be f32 or bf16, got %d", rel_dtype);
  KGE_REQUIRE(ent_dtype != KGE_I8 || ent_scale, KGE_ERR_INVALID, "kge_build_query: int8 entities need ent_scale");
  switch (model) {
    case KGE_DISTMULT: break;
    case KGE_COMPLEX:
      KGE_REQUIRE(d % 2 == 0, KGE_ERR_INVALID, "kge_build_query: ComplEx needs even d, got %lld", (long long)d);
      break;
    case KGE_QMULT:
      KGE_REQUIRE(d % 4 == 0, KGE_ERR_INVALID, "kge_build_query: QMult needs d %% 4 == 0, got %lld", (long long)d);
      break;
    case KGE_OMULT:
      KGE_REQUIRE(d % 8 == 0, KGE_ERR_INVALID, "kge_build_query: OMult needs d %% 8 == 0, got %lld", (long long)d);
      break;
    case KGE_KECI:
      KGE_REQUIRE(p >= 0 && q >= 0 && d % (p + q + 1) == 0, KGE_ERR_INVALID,
                  "kge_build_query: Keci needs d / (p + q + 1) whole, got d=%lld p=%d q=%d", (long long)d, p, q);
      KGE_REQUIRE((p == 0 || coeff_p) && (q == 0 || coeff_q), KGE_ERR_INVALID,
                  "kge_build_query: Keci with p=%d q=%d needs coefficient vectors", p, q);
      KGE_REQUIRE(r == 0, KGE_ERR_INVALID, "kge_build_query: Keci has no degenerate bases (r=%d)", r);
      break;
    case KGE_DECAL:
      KGE_REQUIRE(p >= 0 && q >= 0 && r >= 0 && d % (p + q + r + 1) == 0, KGE_ERR_INVALID,
                  "kge_build_query_decal: needs d / (p + q + r + 1) whole, got d=%lld p=%d q=%d r=%d", (long long)d, p,
                  q, r);
      KGE_REQUIRE((p == 0 || coeff_p) && (q == 0 || coeff_q) && (r == 0 || coeff_r), KGE_ERR_INVALID,
                  "kge_build_query_decal: p=%d q=%d r=%d need their coefficient vectors", p, q, r);
      break;
    default: return set_error(KGE_ERR_INVALID, "kge_build_query: unknown model %d", model);
  }
  QueryArgs a;
  a.ent = ent;
  a.ent_scale = ent_scale;
  a.rel = rel;
  a.coeff_p = coeff_p;
  a.coeff_q = coeff_q;
  a.coeff_r = coeff_r;
  a.hr = hr;
  a.Q = Q;
  a.bias = bias;
  a.norm.kind = KGE_NORM_NONE;
  a.norm.eps = 0.f;
  a.norm.h_a = a.norm.h_b = a.norm.r_a = a.norm.r_b = nullptr;
  if (norm && norm->kind != KGE_NORM_NONE) {
    KGE_REQUIRE(norm->kind == KGE_NORM_LAYERNORM || norm->kind == KGE_NORM_BATCHNORM1D, KGE_ERR_INVALID,
                "kge_build_query: unknown normalisation %d", norm->kind);
    KGE_REQUIRE(norm->h_a && norm->h_b && norm->r_a && norm->r_b, KGE_ERR_INVALID,
                "kge_build_query: normalisation parameters missing");
    a.norm = *norm;
  }
  a.drop = kge_dropout_params{nullptr, nullptr, nullptr, 1.f, 1.f};
  if (dropout) {
    if (int rc = check_dropout("kge_build_query_dropout", dropout, model)) return rc;
    a.drop = *dropout;
  }
  a.B = B;
  a.N = N;
  a.R = R;
  a.d = (int)d;
  a.p = p;
  a.q = q;
  a.r = (model == KGE_DECAL) ? r : 0;
  a.normalize_relation = normalize_relation;
  a.head_mode = head_mode;
  hipStream_t st = (hipStream_t)stream;
  if (ent_dtype == KGE_F32) return launch_build_query<KGE_F32>(a, model, rel_dtype, st);
  if (ent_dtype == KGE_BF16) return launch_build_query<KGE_BF16>(a, model, rel_dtype, st);
  return launch_build_query<KGE_I8>(a, model, rel_dtype, st);
}

extern "C" int kge_build_query(int model, int p, int q, const void* ent, int ent_dtype, const float* ent_scale,
                               const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                               int normalize_relation, const kge_norm_params* norm, const int64_t* hr,
                               int64_t B, int64_t d, int64_t N, int64_t R, float* Q, float* bias, void* stream) {
  if (model == KGE_DECAL)
    return kge::set_error(KGE_ERR_INVALID, "kge_build_query: DeCaL takes three base counts, use kge_build_query_decal");
  return build_query_impl(0, model, p, q, 0, ent, ent_dtype, ent_scale, rel, rel_dtype, coeff_p, coeff_q, nullptr,
                          normalize_relation, norm, hr, B, d, N, R, Q, bias, stream);
}

extern "C" int kge_build_query_head(int model, int p, int q, const void* ent, int ent_dtype, const float* ent_scale,
                                    const void* rel, int rel_dtype, const float* coeff_p, const float* coeff_q,
                                    int normalize_relation, const kge_norm_params* norm, const int64_t* rt,
                                    int64_t B, int64_t d, int64_t N, int64_t R, float* Q, float* bias, void* stream) {
  if (model == KGE_DECAL)
    return kge::set_error(KGE_ERR_INVALID, "kge_build_query_head: DeCaL takes three base counts, use kge_build_query_decal");
  return build_query_impl(1, model, p, q, 0, ent, ent_dtype, ent_scale, rel, rel_dtype, coeff_p, coeff_q, nullptr,
                          normalize_relation, norm, rt, B, d, N, R, Q, bias, stream);
}

extern "C" int kge_build_query_decal(int head, int p, int q, int r, const void* ent, int ent_dtype,
                                     const float* ent_scale, const void* rel, int rel_dtype, const float* coeff_p,
                                     const float* coeff_q, const float* coeff_r, const kge_norm_params* norm,
                                     const int64_t* pairs, int64_t B, int64_t d, int64_t N, int64_t R, float* Q,
                                     float* bias, void* stream) {
  return build_query_impl(head ? 1 : 0, KGE_DECAL, p, q, r, ent, ent_dtype, ent_scale, rel, rel_dtype, coeff_p, coeff_q,
                          coeff_r, 0, norm, pairs, B, d, N, R, Q, bias, stream);
}

extern "C" int kge_build_query_dropout(int model, int p, int q, int r, const void* ent, int ent_dtype,
                                       const float* ent_scale, const void* rel, int rel_dtype, const float* coeff_p,
                                       const float* coeff_q, const float* coeff_r, int normalize_relation,
                                       const kge_norm_params* norm, const kge_dropout_params* dropout,
                                       const int64_t* hr, int64_t B, int64_t d, int64_t N, int64_t R, float* Q,
                                       float* bias, void* stream) {
  return build_query_impl(0, model, p, q, model == KGE_DECAL ? r : 0, ent, ent_dtype, ent_scale, rel, rel_dtype, coeff_p,
                          coeff_q, coeff_r, normalize_relation, norm, hr, B, d, N, R, Q, bias, stream, dropout);
}

extern "C" size_t kge_batchnorm_workspace_bytes(int64_t B, int64_t d);

namespace kge {
namespace {
int build_query_backward_impl(int model, int p, int q, int r, const float* ent, const float* rel, const float* coeff_p,
                              const float* coeff_q, const float* coeff_r, int normalize_relation,
                              const kge_norm_params* norm, const kge_norm_grads* dnorm, const int64_t* hr, int64_t B,
                              int64_t d, int64_t N, int64_t R, const float* dQ, const float* dbias, float* d_ent,
                              float* d_rel, float* d_coeff_p, float* d_coeff_q, float* d_coeff_r, void* stream,
                              const kge_dropout_params* dropout = nullptr, bool batch_stats = false,
                              void* workspace = nullptr, size_t workspace_bytes = 0) {
  clear_error();
  KGE_REQUIRE(B >= 0 && N > 0 && R > 0, KGE_ERR_INVALID, "kge_build_query_backward: B=%lld N=%lld R=%lld", (long long)B,
              (long long)N, (long long)R);
  if (B == 0) return KGE_OK;
  KGE_REQUIRE(ent && rel && hr && dQ && d_ent && d_rel, KGE_ERR_INVALID, "kge_build_query_backward: null pointer argument");
  KGE_REQUIRE(d >= 1 && d <= 8192, KGE_ERR_INVALID, "kge_build_query_backward: d=%lld outside [1, 8192]", (long long)d);
  KGE_REQUIRE(B <= 0x7fffffff, KGE_ERR_INVALID, "kge_build_query_backward: B=%lld too large", (long long)B);
  if (model != KGE_DECAL) r = 0;
  switch (model) {
    case KGE_DISTMULT: break;
    case KGE_COMPLEX:
      KGE_REQUIRE(d % 2 == 0, KGE_ERR_INVALID, "kge_build_query_backward: ComplEx needs even d, got %lld", (long long)d);
      break;
    case KGE_QMULT:
      KGE_REQUIRE(d % 4 == 0, KGE_ERR_INVALID, "kge_build_query_backward: QMult needs d %% 4 == 0, got %lld", (long long)d);
      break;
    case KGE_OMULT:
      KGE_REQUIRE(d % 8 == 0, KGE_ERR_INVALID, "kge_build_query_backward: OMult needs d %% 8 == 0, got %lld", (long long)d);
      break;
    case KGE_KECI:
    case KGE_DECAL:
      KGE_REQUIRE(p >= 0 && q >= 0 && r >= 0 && d % (p + q + r + 1) == 0, KGE_ERR_INVALID,
                  "kge_build_query_backward: needs d / (p + q + r + 1) whole, got d=%lld p=%d q=%d r=%d", (long long)d, p,
                  q, r);
      KGE_REQUIRE((p == 0 || coeff_p) && (q == 0 || coeff_q) && (r == 0 || coeff_r), KGE_ERR_INVALID,
                  "kge_build_query_backward: p=%d q=%d r=%d need their coefficient vectors", p, q, r);
      break;
    default: return set_error(KGE_ERR_INVALID, "kge_build_query_backward: unknown model %d", model);
  }
  QueryBwdArgs a;
  a.ent = ent;
  a.rel = rel;
  a.coeff_p = coeff_p;
  a.coeff_q = coeff_q;
  a.coeff_r = coeff_r;
  a.hr = hr;
  a.dQ = dQ;
  a.dbias = dbias;
  a.d_ent = d_ent;
  a.d_rel = d_rel;
  a.d_coeff_p = d_coeff_p;
  a.d_coeff_q = d_coeff_q;
  a.d_coeff_r = d_coeff_r;
  a.B = B;
  a.N = N;
  a.R = R;
  a.d = (int)d;
  a.p = p;
  a.q = q;
  a.r = r;
  a.normalize_relation = normalize_relation;
  a.norm.kind = KGE_NORM_NONE;
  a.norm.eps = 0.f;
  a.norm.h_a = a.norm.h_b = a.norm.r_a = a.norm.r_b = nullptr;
  a.dn_h_a = a.dn_h_b = a.dn_r_a = a.dn_r_b = nullptr;
  a.dy_h = a.dy_r = nullptr;
  a.drop = kge_dropout_params{nullptr, nullptr, nullptr, 1.f, 1.f};
  if (dropout) {
    if (int rc = check_dropout("kge_build_query_backward", dropout, model)) return rc;
    a.drop = *dropout;
  }
  hipStream_t st = (hipStream_t)stream;
  if (batch_stats) {
    KGE_REQUIRE(norm && norm->kind == KGE_NORM_BATCHNORM1D && norm->h_a && norm->h_b && norm->r_a && norm->r_b,
                KGE_ERR_INVALID,
                "kge_build_query_backward_batchnorm: norm must be BatchNorm1d with the batch's statistics");
    KGE_REQUIRE(d <= 4096, KGE_ERR_UNSUPPORTED, "kge_build_query_backward_batchnorm: d=%lld exceeds 4096", (long long)d);
    KGE_REQUIRE(B >= 2, KGE_ERR_INVALID, "kge_build_query_backward_batchnorm: batch statistics need B >= 2");
    const size_t need = kge_batchnorm_workspace_bytes(B, d);
    KGE_REQUIRE(workspace && workspace_bytes >= need, KGE_ERR_WORKSPACE,
                "kge_build_query_backward_batchnorm: workspace of %zu bytes, need %zu", workspace_bytes, need);
    KGE_REQUIRE(((uintptr_t)workspace & 15) == 0, KGE_ERR_WORKSPACE,
                "kge_build_query_backward_batchnorm: workspace must be 16-byte aligned");
    double* sums = (double*)workspace;
    a.norm = *norm;
    a.dy_h = (float*)(sums + 4 * d);
    a.dy_r = a.dy_h + B * d;
    hipLaunchKernelGGL(bn_zero_kernel, dim3((unsigned)((4 * d + 255) / 256)), dim3(256), 0, st, sums, (int)(4 * d));
    KGE_LAUNCH_CHECK("bn_zero_kernel");
    // (1) the gradients at the normalised rows, (2) their sums over the batch, (3) the gradients at the raw rows
    const size_t lds_bytes = (5 * (size_t)d + (size_t)(d + 3) / 4) * sizeof(float);
    hipLaunchKernelGGL(build_query_backward_kernel<true>, dim3((unsigned)B), dim3(64), lds_bytes, st, a, model);
    KGE_LAUNCH_CHECK("build_query_backward_kernel");
    BnSumArgs sa{ent, rel, hr, a.dy_h, a.dy_r, *norm, a.drop, sums, B, N, R, (int)d};
    const unsigned slices = (unsigned)((B + 63) / 64 < 64 ? (B + 63) / 64 : 64);
    dim3 grid((unsigned)((d + 63) / 64), slices);
    hipLaunchKernelGGL(bn_sums_kernel<true>, grid, dim3(256), 0, st, sa);
    KGE_LAUNCH_CHECK("bn_sums_kernel");
    hipLaunchKernelGGL(bn_backward_apply_kernel, grid, dim3(256), 0, st, sa, d_ent, d_rel);
    KGE_LAUNCH_CHECK("bn_backward_apply_kernel");
    return KGE_OK;
  }
  if (norm && norm->kind != KGE_NORM_NONE) {
    KGE_REQUIRE(norm->kind == KGE_NORM_LAYERNORM || norm->kind == KGE_NORM_BATCHNORM1D, KGE_ERR_INVALID,
                "kge_build_query_backward_norm: unknown normalisation %d", norm->kind);
    KGE_REQUIRE(norm->h_a && norm->h_b && norm->r_a && norm->r_b, KGE_ERR_INVALID,
                "kge_build_query_backward_norm: normalisation parameters missing");
    KGE_REQUIRE(d <= 4096, KGE_ERR_UNSUPPORTED,
                "kge_build_query_backward_norm: d=%lld exceeds 4096 (five rows and a quarter per pair are kept in LDS)",
                (long long)d);
    a.norm = *norm;
    if (dnorm) {
      KGE_REQUIRE(norm->kind == KGE_NORM_LAYERNORM || !(dnorm->h_a || dnorm->h_b || dnorm->r_a || dnorm->r_b),
                  KGE_ERR_INVALID,
                  "kge_build_query_backward_norm: BatchNorm1d(affine=False) has no parameters to take a gradient");
      a.dn_h_a = dnorm->h_a;
      a.dn_h_b = dnorm->h_b;
      a.dn_r_a = dnorm->r_a;
      a.dn_r_b = dnorm->r_b;
    }
    const size_t lds_bytes = (5 * (size_t)d + (size_t)(d + 3) / 4) * sizeof(float);
    hipLaunchKernelGGL(build_query_backward_kernel<true>, dim3((unsigned)B), dim3(64), lds_bytes, st, a, model);
  } else {
    hipLaunchKernelGGL(build_query_backward_kernel<false>, dim3((unsigned)B), dim3(64), 3 * (size_t)d * sizeof(float), st,
                       a, model);
  }
  KGE_LAUNCH_CHECK("build_query_backward_kernel");
  return KGE_OK;
}
}  // namespace
}  // namespace kge

extern "C" size_t kge_batchnorm_workspace_bytes(int64_t B, int64_t d) {
  if (B < 1 || d < 1) return 0;
  return 4 * (size_t)d * sizeof(double) + 2 * (size_t)B * (size_t)d * sizeof(float);
}

extern "C" int kge_batchnorm_stats(const float* ent, const float* rel, const int64_t* hr, int64_t B, int64_t d, int64_t N,
                                   int64_t R, const kge_dropout_params* dropout, float momentum, float* h_mean,
                                   float* h_var, float* r_mean, float* r_var, float* run_h_mean, float* run_h_var,
                                   float* run_r_mean, float* run_r_var, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  using namespace kge;
  clear_error();
  kge_dropout_params drop{nullptr, nullptr, nullptr, 1.f, 1.f};
  if (dropout) {
    if (int rc = check_dropout("kge_batchnorm_stats", dropout, KGE_DISTMULT)) return rc;
    drop = *dropout;
  }
  KGE_REQUIRE(N > 0 && R > 0 && d >= 1 && d <= 8192, KGE_ERR_INVALID, "kge_batchnorm_stats: N=%lld R=%lld d=%lld",
              (long long)N, (long long)R, (long long)d);
  KGE_REQUIRE(B >= 2 && B <= 0x7fffffff, KGE_ERR_INVALID,
              "kge_batchnorm_stats: B=%lld (the statistics of a batch need at least two rows)", (long long)B);
  KGE_REQUIRE(ent && rel && hr && h_mean && h_var && r_mean && r_var, KGE_ERR_INVALID,
              "kge_batchnorm_stats: null pointer argument");
  KGE_REQUIRE(momentum >= 0.f && momentum <= 1.f, KGE_ERR_INVALID, "kge_batchnorm_stats: momentum %g", (double)momentum);
  KGE_REQUIRE(workspace && workspace_bytes >= 4 * (size_t)d * sizeof(double), KGE_ERR_WORKSPACE,
              "kge_batchnorm_stats: workspace of %zu bytes, need %zu", workspace_bytes, 4 * (size_t)d * sizeof(double));
  KGE_REQUIRE(((uintptr_t)workspace & 7) == 0, KGE_ERR_WORKSPACE, "kge_batchnorm_stats: workspace must be 8-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  double* sums = (double*)workspace;
  hipLaunchKernelGGL(bn_zero_kernel, dim3((unsigned)((4 * d + 255) / 256)), dim3(256), 0, st, sums, (int)(4 * d));
  KGE_LAUNCH_CHECK("bn_zero_kernel");
  kge_norm_params none{};
  BnSumArgs sa{ent, rel, hr, nullptr, nullptr, none, drop, sums, B, N, R, (int)d};
  const unsigned slices = (unsigned)((B + 63) / 64 < 64 ? (B + 63) / 64 : 64);
  hipLaunchKernelGGL(bn_sums_kernel<false>, dim3((unsigned)((d + 63) / 64), slices), dim3(256), 0, st, sa);
  KGE_LAUNCH_CHECK("bn_sums_kernel");
  hipLaunchKernelGGL(bn_finish_stats_kernel, dim3((unsigned)((d + 255) / 256)), dim3(256), 0, st, sums, (int)d, B, momentum,
                     h_mean, h_var, r_mean, r_var, run_h_mean, run_h_var, run_r_mean, run_r_var);
  KGE_LAUNCH_CHECK("bn_finish_stats_kernel");
  return KGE_OK;
}

extern "C" int kge_build_query_backward_batchnorm(int model, int p, int q, int r, const float* ent, const float* rel,
                                                  const float* coeff_p, const float* coeff_q, const float* coeff_r,
                                                  int normalize_relation, const kge_norm_params* norm,
                                                  const kge_dropout_params* dropout, const int64_t* hr, int64_t B,
                                                  int64_t d, int64_t N, int64_t R,
                                                  const float* dQ, const float* dbias, float* d_ent, float* d_rel,
                                                  float* d_coeff_p, float* d_coeff_q, float* d_coeff_r,
                                                  void* workspace, size_t workspace_bytes, void* stream) {
  return kge::build_query_backward_impl(model, p, q, r, ent, rel, coeff_p, coeff_q, coeff_r, normalize_relation, norm,
                                        nullptr, hr, B, d, N, R, dQ, dbias, d_ent, d_rel, d_coeff_p, d_coeff_q,
                                        d_coeff_r, stream, dropout, true, workspace, workspace_bytes);
}

extern "C" int kge_build_query_backward(int model, int p, int q, int r, const float* ent, const float* rel,
                                        const float* coeff_p, const float* coeff_q, const float* coeff_r,
                                        int normalize_relation, const int64_t* hr, int64_t B, int64_t d, int64_t N,
                                        int64_t R, const float* dQ, const float* dbias, float* d_ent, float* d_rel,
                                        float* d_coeff_p, float* d_coeff_q, float* d_coeff_r, void* stream) {
  return kge::build_query_backward_impl(model, p, q, r, ent, rel, coeff_p, coeff_q, coeff_r, normalize_relation, nullptr,
                                        nullptr, hr, B, d, N, R, dQ, dbias, d_ent, d_rel, d_coeff_p, d_coeff_q,
                                        d_coeff_r, stream);
}

extern "C" int kge_build_query_backward_norm(int model, int p, int q, int r, const float* ent, const float* rel,
                                             const float* coeff_p, const float* coeff_q, const float* coeff_r,
                                             int normalize_relation, const kge_norm_params* norm,
                                             const kge_norm_grads* dnorm, const kge_dropout_params* dropout,
                                             const int64_t* hr, int64_t B, int64_t d,
                                             int64_t N, int64_t R, const float* dQ, const float* dbias, float* d_ent,
                                             float* d_rel, float* d_coeff_p, float* d_coeff_q, float* d_coeff_r,
                                             void* stream) {
  return kge::build_query_backward_impl(model, p, q, r, ent, rel, coeff_p, coeff_q, coeff_r, normalize_relation, norm,
                                        dnorm, hr, B, d, N, R, dQ, dbias, d_ent, d_rel, d_coeff_p, d_coeff_q, d_coeff_r,
                                        stream, dropout);
}
