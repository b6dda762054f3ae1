// Attention whose scores carry more terms than the product of query and key, and
// whose values may be narrower or wider than its keys.  For the query of head h at
// position p and the key at position j <= p (and, with a window W, j > p - W or j < F, the
// first F positions staying visible beside the window):
//
//   s(p, j) = (q . k) * scale - slope[h] * (p - j)           (slope: optional, one a head)
//   w(p, j) = exp(s(p, j)) / (exp(sink[h]) + sum_j' exp(s(p, j')))
//   out     = gate[row, h] * sum_j w(p, j) v_j                (sink, gate: optional)
//
// With `chunk` C > 0 the key must also lie in the query's run of C positions counted from the
// sequence's start, floor(j / C) = floor(p / C).  With `logistic` the weights are not a softmax:
// w(p, j) = 1 / (1 + exp(-(s(p, j) + score_bias[h]))), every key by itself, no normalisation (and
// no sink).
//
// The sink is a score without a key: it takes part in the normalisation once, is
// neither scaled nor biased, and brings no value.  Scores, weights and the sums over
// values are float whatever the storage type is.
//
// A page of the cache holds the keys of its 64 positions, [kv head][row][dk], and
// behind them the values transposed, [kv head][dv][row].
//
// Also here: the row-wise step between the fused projection and this attention
// (biases, a norm over the whole projection of q and of k, a factor on q that grows
// with the logarithm of the position, the gate's logistic function, and the split),
// and the commit of keys and values of unequal widths to pages.
#include "common.hpp"

namespace tl {

constexpr int SC_MAX_D = 256;

struct ScoreTerms {
  float scale;
  int window;              // 0: none
  int keep_first;          // with a window: positions 0 .. keep_first - 1 stay visible beside it
  const float* slopes;     // [nq] or null
  const float* sinks;      // [nq] or null
  const float* gate;       // [n, nq] or null
  int chunk;               // 0: none; else a key is seen only inside the query's run of `chunk` positions
  int logistic;            // the weights are logistic functions of the scores, not a softmax
  const float* score_bias; // [nq] or null: added to the score (logistic weights only)
};

// One wave per (row, head): the kernel of the 32-bit path and of every shape that the
// matrix-core kernels do not take; the reference the faster ones are checked against.
// TO: the type of the result, T or float (for a caller that goes on in float).
template <typename T, typename TO>
__global__ void __launch_bounds__(64)
attn_scored_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_new, const T* __restrict__ v_new,
                         const T* __restrict__ pages, const int* __restrict__ table, int table_stride,
                         int ring_pages, const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                         const int* __restrict__ cu_seqlens, const int* __restrict__ n_cached, int nq,
                         int nkv, int dk, int dv, ScoreTerms terms, TO* __restrict__ out) {
  __shared__ float q_s[SC_MAX_D];
  __shared__ float p_s[WAVE];
  __shared__ const T* v_s[WAVE];
  __shared__ int vstride_s[WAVE];
  const int n = blockIdx.x / nq, h = blockIdx.x % nq;
  const int lane = threadIdx.x;
  const int b = row_seq[n], p = row_pos[n];
  const int kvh = h / (nq / nkv);
  const int cached = n_cached[b];
  const int row0 = cu_seqlens[b];
  const int window = terms.window;
  int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  if (terms.chunk > 0) lo = max(lo, (p / terms.chunk) * terms.chunk);
  const float sbias = terms.score_bias ? terms.score_bias[h] : 0.f;
  const bool logistic = terms.logistic != 0;
  const size_t keys_elems = (size_t)nkv * PAGE * dk;
  const size_t page_elems = (size_t)nkv * PAGE * (dk + dv);
  const float slope = terms.slopes ? terms.slopes[h] : 0.f;

  const T* qr = q + ((size_t)n * nq + h) * dk;
  for (int i = lane; i < dk; i += WAVE) q_s[i] = to_f32(qr[i]);
  __syncthreads();

  // the sink opens the running sums: a score of its own with weight exp(sink - m) and no value
  float m = terms.sinks ? terms.sinks[h] : -INFINITY;
  float l = terms.sinks ? 1.f : 0.f;
  float acc[SC_MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < SC_MAX_D / WAVE; ++i) acc[i] = 0.f;

  // the keys that are seen: the first ones that stay visible beside the window, then the window
  const int kept = terms.keep_first < lo ? terms.keep_first : lo;
  for (int part = 0; part < 2; ++part) {
  const int begin = part == 0 ? 0 : lo;
  const int end = part == 0 ? kept : p + 1;
  for (int j0 = begin; j0 < end; j0 += WAVE) {
    const int j = j0 + lane;
    float s = -INFINITY;
    const T* vp = nullptr;
    int vstride = 1;                 // values: [dv][PAGE] in a page, [dv] in the step's rows
    if (j < end) {
      const T* kp;
      if (j < cached) {
        const int page = table[(size_t)b * table_stride + (j / PAGE) % ring_pages];
        const T* pg = pages + (size_t)page * page_elems;
        kp = pg + ((size_t)kvh * PAGE + (j % PAGE)) * dk;
        vp = pg + keys_elems + (size_t)kvh * dv * PAGE + (j % PAGE);
        vstride = PAGE;
      } else {
        const size_t r = (size_t)(row0 + j - cached) * nkv + kvh;
        kp = k_new + r * dk;
        vp = v_new + r * dv;
      }
      float dot = 0.f;
      for (int t = 0; t < dk; ++t) dot = fmaf(to_f32(kp[t]), q_s[t], dot);
      s = dot * terms.scale - slope * (float)(p - j) + sbias;
    }
    float pj, alpha;
    if (logistic) {                                   // every key by itself: no maximum, no sum
      pj = (j < end) ? 1.0f / (1.0f + expf(-s)) : 0.f;
      alpha = 1.f;
    } else {
      const float m_new = fmaxf(m, wave_max(s));     // finite: key j0 is visible
      pj = (j < end) ? expf(s - m_new) : 0.f;
      alpha = expf(m - m_new);                        // 0 in the first tile without a sink (m = -inf)
      l = l * alpha + wave_sum(pj);
      m = m_new;
    }
    __syncthreads();
    p_s[lane] = pj;
    v_s[lane] = vp;
    vstride_s[lane] = vstride;
    __syncthreads();
    const int cnt = (end - j0 < WAVE) ? end - j0 : WAVE;
#pragma unroll
    for (int i = 0; i < SC_MAX_D / WAVE; ++i) {
      const int dim = lane + WAVE * i;
      if (dim < dv) {
        float a = acc[i] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a = fmaf(p_s[jj], to_f32(v_s[jj][(size_t)dim * vstride_s[jj]]), a);
        acc[i] = a;
      }
    }
  }
  }
  const float g = terms.gate ? terms.gate[(size_t)n * nq + h] : 1.f;
  TO* o = out + ((size_t)n * nq + h) * dv;
#pragma unroll
  for (int i = 0; i < SC_MAX_D / WAVE; ++i) {
    const int dim = lane + WAVE * i;
    if (dim < dv) o[dim] = from_f32<TO>((logistic ? acc[i] : acc[i] / l) * g);
  }
}

// ---- between the projection and the attention ----------------------------------
// proj[n, :] = [q (nq*dk) | k (nkv*dk) | v (nkv*dv) | g (ng)] in float, k and v absent for a
// mixer that reads another's (nkv == 0).  Per row: add the biases; divide q (all of it, every
// head at once) by its root mean square and multiply by a weight of that size, the same for k;
// multiply q by 1 + coef * ln(floor((pos + 1) / every) + 1); g -> 1 / (1 + exp(-g)).
// k and v go to rows of their own, or (pages != null: one token a sequence) straight into the
// page of the row's position.
struct ProjectionTerms {
  const float* bias;       // [width] or null
  const float* q_norm;     // [nq*dk] or null: no norm
  const float* k_norm;     // [nkv*dk] or null
  float eps;
  float temp_coef;         // 0: no factor
  float temp_every;
};

template <typename T>
__global__ void __launch_bounds__(256)
split_projection_kernel(const float* __restrict__ proj, const int* __restrict__ row_pos, ProjectionTerms t,
                        int nq, int nkv, int dk, int dv, int ng, T* __restrict__ q, T* __restrict__ k,
                        T* __restrict__ v, float* __restrict__ gate, const int* __restrict__ table,
                        int table_stride, int ring_pages, T* __restrict__ pages) {
  __shared__ float sh[4];
  const int n = blockIdx.x;
  const int Q = nq * dk, K = nkv * dk, V = nkv * dv;
  const int width = Q + K + V + ng;
  const float* row = proj + (size_t)n * width;
  const int pos = row_pos[n];

  // q
  float ss = 0.f;
  for (int i = threadIdx.x; i < Q; i += 256) {
    const float a = row[i] + (t.bias ? t.bias[i] : 0.f);
    ss += a * a;
  }
  ss = block_sum<256>(ss, sh);
  float fq = t.q_norm ? 1.0f / sqrtf(ss / (float)Q + t.eps) : 1.f;
  float temp = 1.f;
  if (t.temp_coef != 0.f) {
    const float steps = (float)floor((double)(pos + 1) / (double)t.temp_every);
    temp = 1.0f + t.temp_coef * logf(steps + 1.0f);
  }
  for (int i = threadIdx.x; i < Q; i += 256) {
    float a = row[i] + (t.bias ? t.bias[i] : 0.f);
    a = a * fq;
    if (t.q_norm) a *= t.q_norm[i];
    q[(size_t)n * Q + i] = from_f32<T>(a * temp);
  }
  // gate
  for (int i = threadIdx.x; i < ng; i += 256) {
    const float a = row[Q + K + V + i] + (t.bias ? t.bias[Q + K + V + i] : 0.f);
    gate[(size_t)n * ng + i] = 1.0f / (1.0f + expf(-a));
  }
  if (nkv == 0) return;
  // k
  ss = 0.f;
  for (int i = threadIdx.x; i < K; i += 256) {
    const float a = row[Q + i] + (t.bias ? t.bias[Q + i] : 0.f);
    ss += a * a;
  }
  ss = block_sum<256>(ss, sh);
  const float fk = t.k_norm ? 1.0f / sqrtf(ss / (float)K + t.eps) : 1.f;
  T* kd = nullptr;
  T* vd = nullptr;
  int r = 0;
  if (pages) {
    const int page = table[(size_t)n * table_stride + (pos / PAGE) % ring_pages];
    kd = pages + (size_t)page * nkv * PAGE * (dk + dv);
    vd = kd + (size_t)nkv * PAGE * dk;
    r = pos % PAGE;
  }
  for (int i = threadIdx.x; i < K; i += 256) {
    float a = (row[Q + i] + (t.bias ? t.bias[Q + i] : 0.f)) * fk;
    if (t.k_norm) a *= t.k_norm[i];
    if (pages) kd[((size_t)(i / dk) * PAGE + r) * dk + i % dk] = from_f32<T>(a);
    else k[(size_t)n * K + i] = from_f32<T>(a);
  }
  for (int i = threadIdx.x; i < V; i += 256) {
    const float a = row[Q + K + i] + (t.bias ? t.bias[Q + K + i] : 0.f);
    if (pages) vd[((size_t)(i / dv) * dv + i % dv) * PAGE + r] = from_f32<T>(a);
    else v[(size_t)n * V + i] = from_f32<T>(a);
  }
}

// The same, four channels at a time and three workgroups a row (blockIdx.y: q and the gate, k, v):
// few rows, as in single-token steps, otherwise wait for one workgroup's chain of loads each.  All
// of nq*dk, nkv*dk, nkv*dv and dk are multiples of 4 and the buffers 16-byte aligned.
__device__ __forceinline__ float4 ld_f4(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <typename T> __device__ __forceinline__ void st4(T* p, float4 a);
template <> __device__ __forceinline__ void st4<float>(float* p, float4 a) { *reinterpret_cast<float4*>(p) = a; }
template <> __device__ __forceinline__ void st4<bf16>(bf16* p, float4 a) {
  bf16x4 o;
  o[0] = (bf16)a.x; o[1] = (bf16)a.y; o[2] = (bf16)a.z; o[3] = (bf16)a.w;
  *reinterpret_cast<bf16x4*>(p) = o;
}

template <typename T>
__global__ void __launch_bounds__(256)
split_projection_vec_kernel(const float* __restrict__ proj, const int* __restrict__ row_pos, ProjectionTerms t,
                            int nq, int nkv, int dk, int dv, int ng, T* __restrict__ q, T* __restrict__ k,
                            T* __restrict__ v, float* __restrict__ gate, const int* __restrict__ table,
                            int table_stride, int ring_pages, T* __restrict__ pages) {
  __shared__ float sh[4];
  const int n = blockIdx.x, section = blockIdx.y;
  const int Q = nq * dk, K = nkv * dk, V = nkv * dv;
  const float* row = proj + (size_t)n * (Q + K + V + ng);
  const int pos = row_pos[n];
  // a piece of the row with its bias
  auto piece = [&](int off, int c) {
    float4 a = ld_f4(row + off + 4 * c);
    if (t.bias) {
      const float4 b = ld_f4(t.bias + off + 4 * c);
      a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    return a;
  };
  auto mean_square = [&](int off, int len) {
    float ss = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < len / 4; c += 256) {
      const float4 a = piece(off, c);
      ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
    }
    return block_sum<256>(ss, sh) / (float)len;
  };
  if (section == 0) {
    float f = t.q_norm ? 1.0f / sqrtf(mean_square(0, Q) + t.eps) : 1.f;
    float temp = 1.f;
    if (t.temp_coef != 0.f) {
      const float steps = (float)floor((double)(pos + 1) / (double)t.temp_every);
      temp = 1.0f + t.temp_coef * logf(steps + 1.0f);
    }
#pragma unroll 4
    for (int c = threadIdx.x; c < Q / 4; c += 256) {
      float4 a = piece(0, c);
      a.x *= f; a.y *= f; a.z *= f; a.w *= f;
      if (t.q_norm) {
        const float4 w = ld_f4(t.q_norm + 4 * c);
        a.x *= w.x; a.y *= w.y; a.z *= w.z; a.w *= w.w;
      }
      a.x *= temp; a.y *= temp; a.z *= temp; a.w *= temp;
      st4<T>(q + (size_t)n * Q + 4 * c, a);
    }
    for (int i = threadIdx.x; i < ng; i += 256) {
      const float a = row[Q + K + V + i] + (t.bias ? t.bias[Q + K + V + i] : 0.f);
      gate[(size_t)n * ng + i] = 1.0f / (1.0f + expf(-a));
    }
    return;
  }
  T* kd = nullptr;
  T* vd = nullptr;
  int r = 0;
  if (pages) {
    const int page = table[(size_t)n * table_stride + (pos / PAGE) % ring_pages];
    kd = pages + (size_t)page * nkv * PAGE * (dk + dv);
    vd = kd + (size_t)nkv * PAGE * dk;
    r = pos % PAGE;
  }
  if (section == 1) {
    const float f = t.k_norm ? 1.0f / sqrtf(mean_square(Q, K) + t.eps) : 1.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < K / 4; c += 256) {
      float4 a = piece(Q, c);
      a.x *= f; a.y *= f; a.z *= f; a.w *= f;
      if (t.k_norm) {
        const float4 w = ld_f4(t.k_norm + 4 * c);
        a.x *= w.x; a.y *= w.y; a.z *= w.z; a.w *= w.w;
      }
      const int i = 4 * c;
      if (pages) st4<T>(kd + ((size_t)(i / dk) * PAGE + r) * dk + i % dk, a);
      else st4<T>(k + (size_t)n * K + i, a);
    }
    return;
  }
#pragma unroll 4
  for (int c = threadIdx.x; c < V / 4; c += 256) {
    const float4 a = piece(Q + K, c);
    const int i = 4 * c;
    if (pages) {
      const float e[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int u = 0; u < 4; ++u) vd[((size_t)((i + u) / dv) * dv + (i + u) % dv) * PAGE + r] = from_f32<T>(e[u]);
    } else {
      st4<T>(v + (size_t)n * V + i, a);
    }
  }
}

// Rows of keys [n, nkv, dk] and values [n, nkv, dv] into the pages of their positions.  A row
// that the same step overwrites in a ring (older than the ring is long) is skipped.
template <typename T>
__global__ void kv_commit_wide_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                      const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                                      const int* __restrict__ len_after, const int* __restrict__ table,
                                      int table_stride, int ring_pages, int nkv, int dk, int dv,
                                      T* __restrict__ pages) {
  const int n = blockIdx.x;
  const int b = row_seq[n], p = row_pos[n];
  if ((long long)p < (long long)len_after[b] - (long long)ring_pages * PAGE) return;
  const int page = table[(size_t)b * table_stride + (p / PAGE) % ring_pages];
  const int r = p % PAGE;
  T* kd = pages + (size_t)page * nkv * PAGE * (dk + dv);
  T* vd = kd + (size_t)nkv * PAGE * dk;
  const T* ks = k + (size_t)n * nkv * dk;
  const T* vs = v + (size_t)n * nkv * dv;
  for (int t = threadIdx.x; t < nkv * dk; t += blockDim.x)
    kd[((size_t)(t / dk) * PAGE + r) * dk + t % dk] = ks[t];
  for (int t = threadIdx.x; t < nkv * dv; t += blockDim.x)
    vd[((size_t)(t / dv) * dv + t % dv) * PAGE + r] = vs[t];
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_attn_scored_plain(const void* q, const void* k_new, const void* v_new, const void* pages, int dt,
                         const int* table, int table_stride, int ring_pages, const int* row_seq,
                         const int* row_pos, const int* cu_seqlens, const int* n_cached, int n, int nq,
                         int nkv, int dk, int dv, int window, int keep_first, int chunk, float scale, const float* slopes,
                         const float* sinks, const float* gate, int logistic, const float* score_bias, void* out, int out_dt,
                         hipStream_t st) {
  TL_REQUIRE(chunk >= 0 && (!logistic || sinks == nullptr) && (logistic || score_bias == nullptr),
             "scored attention: %d positions a chunk; logistic weights have no sink, a softmax no bias on the score", chunk);
  TL_REQUIRE(out_dt == dt || out_dt == DT_F32, "scored attention: the result is of the operands' type or float");
  TL_REQUIRE(n >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "scored attention: bad head counts nq=%d nkv=%d",
             nq, nkv);
  TL_REQUIRE(dk > 0 && dk <= SC_MAX_D && dv > 0 && dv <= SC_MAX_D,
             "scored attention: head sizes %d and %d are not served (1..%d)", dk, dv, SC_MAX_D);
  TL_REQUIRE(ring_pages > 0 && table_stride > 0 && window >= 0 && keep_first >= 0,
             "scored attention: bad cache geometry ring_pages=%d table_stride=%d window=%d keep_first=%d", ring_pages,
             table_stride, window, keep_first);
  TL_REQUIRE(keep_first == 0 || window == 0 || (long long)ring_pages * PAGE >= (1LL << 24),
             "scored attention: first positions that stay visible beside a window need a cache that keeps every position");
  TL_REQUIRE((long long)n * nq < 2147483647LL, "scored attention: too many (row, head) pairs");
  if (n == 0) return 0;
  const ScoreTerms terms{scale, window, window > 0 ? keep_first : 0, slopes, sinks, gate, chunk, logistic, score_bias};
  if (dt == DT_F32)
    attn_scored_plain_kernel<float, float><<<n * nq, 64, 0, st>>>(
        (const float*)q, (const float*)k_new, (const float*)v_new, (const float*)pages, table, table_stride,
        ring_pages, row_seq, row_pos, cu_seqlens, n_cached, nq, nkv, dk, dv, terms, (float*)out);
  else if (dt == DT_BF16 && out_dt == DT_F32)
    attn_scored_plain_kernel<bf16, float><<<n * nq, 64, 0, st>>>(
        (const bf16*)q, (const bf16*)k_new, (const bf16*)v_new, (const bf16*)pages, table, table_stride,
        ring_pages, row_seq, row_pos, cu_seqlens, n_cached, nq, nkv, dk, dv, terms, (float*)out);
  else if (dt == DT_BF16)
    attn_scored_plain_kernel<bf16, bf16><<<n * nq, 64, 0, st>>>(
        (const bf16*)q, (const bf16*)k_new, (const bf16*)v_new, (const bf16*)pages, table, table_stride,
        ring_pages, row_seq, row_pos, cu_seqlens, n_cached, nq, nkv, dk, dv, terms, (bf16*)out);
  else
    TL_REQUIRE(false, "scored attention: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("attn_scored_plain");
  return 0;
}

// pages null: k and v go to the rows `k`, `v`; else (one token a sequence, row n is sequence n)
// into the pages.  nkv 0: the projection holds q and g alone.
int tl_split_projection(const float* proj, const int* row_pos, const float* bias, const float* q_norm,
                        const float* k_norm, float eps, float temp_coef, float temp_every, int n, int nq,
                        int nkv, int dk, int dv, int ng, void* q, void* k, void* v, float* gate, int dt,
                        const int* table, int table_stride, int ring_pages, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv >= 0 && dk > 0 && dv > 0 && ng >= 0,
             "split_projection: bad sizes n=%d nq=%d nkv=%d dk=%d dv=%d ng=%d", n, nq, nkv, dk, dv, ng);
  TL_REQUIRE(ng == 0 || gate != nullptr, "split_projection: %d gate channels and nowhere to put them", ng);
  TL_REQUIRE(nkv == 0 || pages != nullptr || (k != nullptr && v != nullptr),
             "split_projection: keys and values need rows or pages to go to");
  TL_REQUIRE(pages == nullptr || (table != nullptr && table_stride > 0 && ring_pages > 0),
             "split_projection: pages without a page table");
  TL_REQUIRE(temp_coef == 0.f || temp_every > 0.f, "split_projection: the factor on q needs a positive step");
  if (n == 0) return 0;
  const ProjectionTerms t{bias, q_norm, k_norm, eps, temp_coef, temp_every};
  const int Q = nq * dk, K = nkv * dk, V = nkv * dv;
  auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  const bool vec = Q % 4 == 0 && K % 4 == 0 && V % 4 == 0 && dk % 4 == 0 && ng % 4 == 0 && al(proj) && al(bias) &&
                   al(q_norm) && al(k_norm) && al(q) && al(k) && al(v) && al(pages);
  if (vec && (dt == DT_F32 || dt == DT_BF16)) {
    const dim3 grid(n, nkv > 0 ? 3 : 1);
    if (dt == DT_F32)
      split_projection_vec_kernel<float><<<grid, 256, 0, st>>>(proj, row_pos, t, nq, nkv, dk, dv, ng, (float*)q, (float*)k,
                                                               (float*)v, gate, table, table_stride, ring_pages, (float*)pages);
    else
      split_projection_vec_kernel<bf16><<<grid, 256, 0, st>>>(proj, row_pos, t, nq, nkv, dk, dv, ng, (bf16*)q, (bf16*)k,
                                                              (bf16*)v, gate, table, table_stride, ring_pages, (bf16*)pages);
    TL_LAUNCH_CHECK("split_projection");
    return 0;
  }
  if (dt == DT_F32)
    split_projection_kernel<float><<<n, 256, 0, st>>>(proj, row_pos, t, nq, nkv, dk, dv, ng, (float*)q, (float*)k,
                                                     (float*)v, gate, table, table_stride, ring_pages, (float*)pages);
  else if (dt == DT_BF16)
    split_projection_kernel<bf16><<<n, 256, 0, st>>>(proj, row_pos, t, nq, nkv, dk, dv, ng, (bf16*)q, (bf16*)k,
                                                    (bf16*)v, gate, table, table_stride, ring_pages, (bf16*)pages);
  else
    TL_REQUIRE(false, "split_projection: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("split_projection");
  return 0;
}

int tl_kv_commit_wide(const void* k, const void* v, int dt, const int* row_seq, const int* row_pos,
                      const int* len_after, const int* table, int table_stride, int ring_pages, int n,
                      int nkv, int dk, int dv, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nkv > 0 && dk > 0 && dv > 0 && ring_pages > 0 && table_stride > 0,
             "kv_commit_wide: bad sizes n=%d nkv=%d dk=%d dv=%d", n, nkv, dk, dv);
  if (n == 0) return 0;
  const int nt = nkv * (dk > dv ? dk : dv) >= 256 ? 256 : 64;
  if (dt == DT_F32)
    kv_commit_wide_kernel<float><<<n, nt, 0, st>>>((const float*)k, (const float*)v, row_seq, row_pos, len_after,
                                                    table, table_stride, ring_pages, nkv, dk, dv, (float*)pages);
  else if (dt == DT_BF16)
    kv_commit_wide_kernel<bf16><<<n, nt, 0, st>>>((const bf16*)k, (const bf16*)v, row_seq, row_pos, len_after,
                                                   table, table_stride, ring_pages, nkv, dk, dv, (bf16*)pages);
  else
    TL_REQUIRE(false, "kv_commit_wide: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("kv_commit_wide");
  return 0;
}

}  // extern "C"
