// Between the fused projection of an attention and the attention itself, head by head.
//
// A row of the projection is [q (nq*dk) | k (nkv*dk) | v (nkv*dv) | g (ng)] in float.  Per row:
//
//   * the biases are added (optional);
//   * every head of q and of k is divided by ITS OWN root mean square over its dk channels,
//     eps inside the root, and multiplied by a weight of dk channels that all heads share
//     (optional; q and k have a weight each);
//   * the first `rotary_dim` channels of every head of q and k are rotated in pairs
//     (i, i + rotary_dim/2) by the angle pos * inv_freq[i];
//   * or (`unit_norm`) every head of q and of k is divided by its root mean square AFTER the
//     rotation, with no weight;
//   * the values are mixed with those that an earlier layer left for the same row:
//     v <- (1 - lambda) v + lambda v_first  (`mix` 2), or are left for later layers (`mix` 1);
//     v_first is float, unrounded;
//   * g -> 1 / (1 + exp(-g)), one gate per channel of the concatenated heads (ng = nq*dv) or
//     any other number.
//
// k and v go to rows of their own, or (pages != null: one token a sequence) straight into the
// page of the row's position; a mixer that reads another's keys and values has none of its own
// (nkv == 0: the row is [q | g]).  One wave takes one unit of work: a head of q, a head of k, a
// head of v, or 256 gate channels.
#include "common.hpp"

namespace tl {

constexpr int HP_MAX_D = 256;

struct HeadTerms {
  const float* bias;       // [Q + K + V + ng] or null
  const float* q_norm;     // [dk] or null
  const float* k_norm;     // [dk] or null
  float eps;
  int mix;                 // 0: none; 1: leave v in v_first; 2: mix with v_first
  float lambda;
  float* v_first;          // [n, nkv*dv] float
  int unit_norm;           // q and k heads divided by their root mean square after the rotation, no weight
};

template <typename T>
__global__ void __launch_bounds__(256)
head_prepare_kernel(const float* __restrict__ proj, const int* __restrict__ row_pos, Rotation rot, HeadTerms t,
                    int nq, int nkv, int dk, int dv, int ng, T* __restrict__ q, T* __restrict__ k, T* __restrict__ v,
                    float* __restrict__ gate, const int* __restrict__ table, int table_stride, int ring_pages,
                    T* __restrict__ pages) {
  const int n = blockIdx.x;
  const int lane = threadIdx.x % WAVE;
  const int unit = blockIdx.y * 4 + threadIdx.x / WAVE;
  const int Q = nq * dk, K = nkv * dk, V = nkv * dv;
  const int gate_units = (ng + 255) / 256;
  if (unit >= nq + 2 * nkv + gate_units) return;
  const float* row = proj + (size_t)n * (Q + K + V + ng);
  const int pos = row_pos[n];
  auto at = [&](int i) { return row[i] + (t.bias ? t.bias[i] : 0.f); };

  int r = 0;
  T* kd = nullptr;
  T* vd = nullptr;
  if (pages && unit >= nq && unit < nq + 2 * nkv) {
    const int page = table[(size_t)n * table_stride + (pos / PAGE) % ring_pages];
    kd = pages + (size_t)page * nkv * PAGE * (dk + dv);
    vd = kd + (size_t)nkv * PAGE * dk;
    r = pos % PAGE;
  }

  if (unit < nq + nkv) {                       // a head of q or of k
    const bool is_q = unit < nq;
    const int head = is_q ? unit : unit - nq;
    const int off = (is_q ? 0 : Q) + head * dk;
    const float* w = is_q ? t.q_norm : t.k_norm;
    float f = 1.f;
    if (w) {
      float ss = 0.f;
      for (int c = lane; c < dk; c += WAVE) {
        const float a = at(off + c);
        ss += a * a;
      }
      ss = wave_sum(ss);
      f = 1.0f / sqrtf(ss / (float)dk + t.eps);
    }
    auto val = [&](int c) {
      float a = at(off + c) * f;
      if (w) a *= w[c];
      return a;
    };
    const int half = rot.rotary_dim / 2;
    auto rotated = [&](int c) {
      if (c >= 2 * half) return val(c);
      const int i = c < half ? c : c - half;
      float sn, cs, ra, rb;
      sincosf((float)pos * rot.inv_freq[i], &sn, &cs);
      rotate_pair(val(i), val(i + half), cs, sn, ra, rb);
      return c < half ? ra : rb;
    };
    float after = 1.f;
    if (t.unit_norm) {
      float ss = 0.f;
      for (int c = lane; c < dk; c += WAVE) {
        const float a = rotated(c);
        ss += a * a;
      }
      after = 1.0f / sqrtf(wave_sum(ss) / (float)dk + t.eps);
    }
    for (int c = lane; c < dk; c += WAVE) {
      const float a = rotated(c) * after;
      const T o = from_f32<T>(a);
      if (is_q) q[(size_t)n * Q + head * dk + c] = o;
      else if (pages) kd[((size_t)head * PAGE + r) * dk + c] = o;
      else k[(size_t)n * K + head * dk + c] = o;
    }
    return;
  }
  if (unit < nq + 2 * nkv) {                   // a head of v
    const int head = unit - nq - nkv;
    for (int c = lane; c < dv; c += WAVE) {
      const int i = head * dv + c;
      float a = at(Q + K + i);
      if (t.mix == 1) t.v_first[(size_t)n * V + i] = a;
      else if (t.mix == 2) a = (1.0f - t.lambda) * a + t.lambda * t.v_first[(size_t)n * V + i];
      const T o = from_f32<T>(a);
      if (pages) vd[((size_t)head * dv + c) * PAGE + r] = o;
      else v[(size_t)n * V + i] = o;
    }
    return;
  }
  const int g0 = (unit - nq - 2 * nkv) * 256;  // gate channels
  for (int i = g0 + lane; i < min(ng, g0 + 256); i += WAVE)
    gate[(size_t)n * ng + i] = 1.0f / (1.0f + expf(-at(Q + K + V + i)));
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_head_prepare(const float* proj, const int* row_pos, const float* inv_freq, int rotary_dim, const float* bias,
                    const float* q_norm, const float* k_norm, float eps, int unit_norm, int mix, float lambda, float* v_first,
                    int n, int nq, int nkv, int dk, int dv, int ng, void* q, void* k, void* v, float* gate, int dt,
                    const int* table, int table_stride, int ring_pages, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv >= 0 && dk > 0 && dv > 0 && ng >= 0 && dk <= HP_MAX_D && dv <= HP_MAX_D,
             "head_prepare: bad sizes n=%d nq=%d nkv=%d dk=%d dv=%d ng=%d (heads up to %d)", n, nq, nkv, dk, dv, ng, HP_MAX_D);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim % 2 == 0 && rotary_dim <= dk,
             "head_prepare: %d rotated channels of a head of %d (even, at most the head)", rotary_dim, dk);
  TL_REQUIRE(rotary_dim == 0 || inv_freq, "head_prepare: a rotation without frequencies");
  TL_REQUIRE(proj && row_pos && q && (nkv == 0 || pages || (k && v)), "head_prepare: a buffer is missing");
  TL_REQUIRE(!unit_norm || (q_norm == nullptr && k_norm == nullptr), "head_prepare: a norm before the rotation or one after it");
  TL_REQUIRE(ng == 0 || gate, "head_prepare: %d gate channels and nowhere to put them", ng);
  TL_REQUIRE(mix >= 0 && mix <= 2 && (mix == 0 || v_first), "head_prepare: mixing values needs the buffer they are left in");
  TL_REQUIRE(pages == nullptr || (table && table_stride > 0 && ring_pages > 0), "head_prepare: pages without a page table");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "head_prepare: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const Rotation rot{inv_freq, rotary_dim, 0};
  const HeadTerms t{bias, q_norm, k_norm, eps, mix, lambda, v_first, unit_norm};
  const int units = nq + 2 * nkv + (ng + 255) / 256;
  const dim3 grid(n, (units + 3) / 4);
  if (dt == DT_F32)
    head_prepare_kernel<float><<<grid, 256, 0, st>>>(proj, row_pos, rot, t, nq, nkv, dk, dv, ng, (float*)q, (float*)k,
                                                     (float*)v, gate, table, table_stride, ring_pages, (float*)pages);
  else
    head_prepare_kernel<bf16><<<grid, 256, 0, st>>>(proj, row_pos, rot, t, nq, nkv, dk, dv, ng, (bf16*)q, (bf16*)k,
                                                    (bf16*)v, gate, table, table_stride, ring_pages, (bf16*)pages);
  TL_LAUNCH_CHECK("head_prepare");
  return 0;
}

}  // extern "C"
