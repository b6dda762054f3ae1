// A routed mixture of small feed-forward layers ("experts").
//
// Router, per row, in float: z = W_r h, s = softmax(z) over all E experts (or, `logistic`, every
// expert's own 1 / (1 + exp(-z))).  The experts form
// `groups` equal groups of neighbours; a group's score is its largest s, and only experts of the
// `keep` best groups can be chosen (groups == 0: every expert can).  Of those the `top` with the
// largest s are chosen; their weights are their s, not renormalised.  Of equal scores the one
// with the smaller index goes first.
//
// `route` leaves the weights as a row of E floats, zero for an expert that was not chosen.
// The experts run as ONE wide feed-forward: the rows of all up projections stacked (the shared
// expert's behind them), the activation times the row's weight of the column's expert
// (`expert_act`), and all down projections side by side: an expert with weight zero adds nothing.
// Steps of few rows run the chosen experts alone instead (`expert_rows_up`, `expert_rows_down`).
#include "common.hpp"

namespace tl {

constexpr int RT_MAX_E = 1024;

// NT threads a row: a quarter of a thousand, or 1024 for steps of few rows, where a row's dots are what the step waits
// for (16 waves take 16 experts at a time instead of 4).  A dot is one wave's either way: the same bits.
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
route_kernel(const T* __restrict__ h, int W, const float* __restrict__ wr, int E, int groups, int keep, int top,
             int logistic, float* __restrict__ weights, int* __restrict__ chosen, bool vec) {
  __shared__ float s_s[RT_MAX_E];
  __shared__ float g_s[RT_MAX_E];
  __shared__ unsigned char ok_s[RT_MAX_E];
  __shared__ float sh[NT / WAVE];
  const int n = blockIdx.x;
  const int t = threadIdx.x, lane = t % WAVE, wave = t / WAVE;
  const T* row = h + (size_t)n * W;
  for (int e = wave; e < E; e += NT / WAVE) {
    const float* w = wr + (size_t)e * W;
    float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;      // four chains: the loads of one do not wait for another's sum
    int c = 0;
    if (vec) {                                         // four channels a lane and load
#pragma unroll 4
      for (c = lane * 4; c + 3 < W; c += WAVE * 4) {
        const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c);
        float r0, r1, r2, r3;
        if constexpr (sizeof(T) == 2) {
          const bf16x4 rv = *reinterpret_cast<const bf16x4*>(row + c);
          r0 = (float)rv[0], r1 = (float)rv[1], r2 = (float)rv[2], r3 = (float)rv[3];
        } else {
          const f32x4 rv = *reinterpret_cast<const f32x4*>(row + c);
          r0 = rv[0], r1 = rv[1], r2 = rv[2], r3 = rv[3];
        }
        d0 = fmaf(wv[0], r0, d0);
        d1 = fmaf(wv[1], r1, d1);
        d2 = fmaf(wv[2], r2, d2);
        d3 = fmaf(wv[3], r3, d3);
      }
    } else {
      for (c = lane; c < W; c += WAVE) d0 = fmaf(w[c], to_f32(row[c]), d0);
    }
    float dot = wave_sum((d0 + d1) + (d2 + d3));
    if (lane == 0) s_s[e] = dot;
  }
  __syncthreads();
  if (logistic) {                                      // every expert's score by itself
    for (int e = t; e < E; e += NT) s_s[e] = 1.0f / (1.0f + expf(-s_s[e]));
  } else {
    float m = -INFINITY;
    for (int e = t; e < E; e += NT) m = fmaxf(m, s_s[e]);
    m = block_max<NT>(m, sh);
    float sum = 0.f;
    for (int e = t; e < E; e += NT) sum += expf(s_s[e] - m);
    sum = block_sum<NT>(sum, sh);
    __syncthreads();
    for (int e = t; e < E; e += NT) s_s[e] = expf(s_s[e] - m) / sum;
  }
  __syncthreads();
  if (groups > 0) {
    const int per = E / groups;
    for (int g = t; g < groups; g += NT) {
      float best = s_s[g * per];
      for (int i = 1; i < per; ++i) best = fmaxf(best, s_s[g * per + i]);
      g_s[g] = best;
    }
    __syncthreads();
    for (int g = t; g < groups; g += NT) {
      int ahead = 0;
      const float mine = g_s[g];
      for (int o = 0; o < groups; ++o) ahead += (g_s[o] > mine || (g_s[o] == mine && o < g)) ? 1 : 0;
      for (int i = 0; i < per; ++i) ok_s[g * per + i] = ahead < keep;
    }
  } else {
    for (int e = t; e < E; e += NT) ok_s[e] = 1;
  }
  __syncthreads();
  for (int e = t; e < E; e += NT) {
    float wgt = 0.f;
    if (ok_s[e]) {
      int ahead = 0;
      const float mine = s_s[e];
      for (int o = 0; o < E; ++o) ahead += (ok_s[o] && (s_s[o] > mine || (s_s[o] == mine && o < e))) ? 1 : 0;
      if (ahead < top) {
        wgt = mine;
        if (chosen) chosen[(size_t)n * top + ahead] = e;
      }
    }
    weights[(size_t)n * E + e] = wgt;
  }
}

// out[n, j] = act(u[n, j]) * (j < E * ff ? weights[n, j / ff] : 1), act = the square of max(., 0)
// (code 0) or max(., 0) (code 1).
template <typename T>
__global__ void __launch_bounds__(256)
expert_act_kernel(const float* __restrict__ u, const float* __restrict__ weights, int E, int ff, int total, int act,
                  T* __restrict__ out) {
  const int n = blockIdx.x;
  for (int j = blockIdx.y * 256 + threadIdx.x; j < total; j += gridDim.y * 256) {
    float a = fmaxf(u[(size_t)n * total + j], 0.f);
    if (act == 0) a *= a;
    if (j < E * ff) a *= weights[(size_t)n * E + j / ff];
    out[(size_t)n * total + j] = from_f32<T>(a);
  }
}


// ---- the chosen experts alone, row by row ---------------------------------------------------------------
// For steps of few rows (fewer chosen experts than there are experts) the wide feed-forward would read every
// expert's weights to use a few: here a row reads the weights of its own `top` experts and of the shared one,
// as two products of a matrix with a vector each.  up [E * ff + shared, H] and down [H, E * ff + shared] are
// the stacked matrices of the wide form, row-major.  Slot k < top of row n is expert chosen[n, k] with the
// router's weight, slot `top` (with a shared expert) is the shared one with weight 1.

// sum_i a[i] * b[i] over one wave; `vec`: both rows are aligned for loads of 16 bytes and len is a multiple of
// the vector's length
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ a, const T* __restrict__ b, int len, bool vec, int lane) {
  float acc = 0.f;
  if (vec) {
    if constexpr (sizeof(T) == 2) {
      for (int i = lane * 8; i < len; i += WAVE * 8) {
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(a + i);
        const bf16x8 y = *reinterpret_cast<const bf16x8*>(b + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc = fmaf((float)x[j], (float)y[j], acc);
      }
    } else {
      for (int i = lane * 4; i < len; i += WAVE * 4) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(a + i);
        const f32x4 y = *reinterpret_cast<const f32x4*>(b + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = fmaf(x[j], y[j], acc);
      }
    }
  } else {
    for (int i = lane; i < len; i += WAVE) acc = fmaf(to_f32(a[i]), to_f32(b[i]), acc);
  }
  return wave_sum(acc);
}

constexpr int ER_ROWS = 16;      // outputs of a workgroup: four a wave

// hs[n, k * ff + j] = act(up[e_k * ff + j] . y[n]) * s[n, e_k];  hs[n, top * ff + j] = act(up[E * ff + j] . y[n])
template <typename T>
__global__ void __launch_bounds__(256)
expert_rows_up_kernel(const T* __restrict__ y, int H, const T* __restrict__ up, const int* __restrict__ chosen,
                      const float* __restrict__ weights, int E, int top, int ff, int shared, int act, bool vec,
                      T* __restrict__ hs) {
  const int slots = top + (shared ? 1 : 0);
  const int n = blockIdx.x / slots, k = blockIdx.x % slots;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  int base, count;
  float scale = 1.f;
  if (k < top) {
    const int e = chosen[(size_t)n * top + k];
    base = e * ff;
    count = ff;
    scale = weights[(size_t)n * E + e];
  } else {
    base = E * ff;
    count = shared;
  }
  const T* row = y + (size_t)n * H;
  T* out = hs + (size_t)n * (top * ff + shared) + (size_t)k * ff;
#pragma unroll
  for (int r = 0; r < ER_ROWS / 4; ++r) {
    const int j = blockIdx.y * ER_ROWS + wave * (ER_ROWS / 4) + r;
    if (j >= count) break;
    float a = fmaxf(wave_dot(up + (size_t)(base + j) * H, row, H, vec, lane), 0.f);
    if (act == 0) a *= a;
    if (lane == 0) out[j] = from_f32<T>(a * scale);
  }
}

// out[n, c] (+)= sum over the row's slots of down[c, slot's columns] . hs[n, slot's part]
template <typename T>
__global__ void __launch_bounds__(256)
expert_rows_down_kernel(const T* __restrict__ hs, const T* __restrict__ down, const int* __restrict__ chosen, int E, int top,
                        int ff, int shared, int H, bool vec, int accumulate, float* __restrict__ out) {
  const int n = blockIdx.x;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const int total = E * ff + shared;
  const T* h = hs + (size_t)n * (top * ff + shared);
#pragma unroll
  for (int r = 0; r < ER_ROWS / 4; ++r) {
    const int c = blockIdx.y * ER_ROWS + wave * (ER_ROWS / 4) + r;
    if (c >= H) break;
    const T* w = down + (size_t)c * total;
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc += wave_dot(w + (size_t)chosen[(size_t)n * top + k] * ff, h + (size_t)k * ff, ff, vec, lane);
    if (shared) acc += wave_dot(w + (size_t)E * ff, h + (size_t)top * ff, shared, vec, lane);
    if (lane == 0) {
      float* o = out + (size_t)n * H + c;
      *o = accumulate ? *o + acc : acc;
    }
  }
}


// ---- gated experts ----------------------------------------------------------------------------------------
// An expert with a gate: down(act(g, u)) with g = W_gate t, u = W_up t and
//     act(g, u) = g' logistic(alpha g') (u' + shift) ,  g' = min(g, limit) ,  u' = clamp(u, -limit, limit).
// The stacked matrix holds, expert after expert, the rows [gate (ff) | up (ff)], and behind the last expert
// the shared one's [gate (shared) | up (shared)], which has a limit of its own.  The router's weight s
// multiplies the expert's INPUT t = s y (`on_input`: g and u are linear in t, so s multiplies both before
// the clamps) or its output (the activation times s).  An expert with weight 0 adds nothing either way.
struct GateTerms {
  float limit, limit_shared, alpha, shift;
  int on_input;
};

__device__ __forceinline__ float gated_value(float g, float u, float s, float limit, const GateTerms& k) {
  if (k.on_input) {
    g *= s;
    u *= s;
  }
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  const float a = g / (1.0f + expf(-k.alpha * g)) * (u + k.shift);
  return k.on_input ? a : a * s;
}

// out[n, j] for the E * ff + shared hidden channels j; gu float [n, 2 (E * ff + shared)] as the stacked matrix
// lays it; weights [n, E] (E == 0: none; a column of weight 1 for the shared part)
template <typename T>
__global__ void __launch_bounds__(256)
expert_gated_act_kernel(const float* __restrict__ gu, const float* __restrict__ weights, int E, int ff, int shared,
                        GateTerms k, T* __restrict__ out) {
  const int n = blockIdx.x;
  const int total = E * ff + shared;
  const float* row = gu + (size_t)n * 2 * total;
  for (int j = blockIdx.y * 256 + threadIdx.x; j < total; j += gridDim.y * 256) {
    float a;
    if (j < E * ff) {
      const int e = j / ff, c = j % ff;
      a = gated_value(row[2 * e * ff + c], row[2 * e * ff + ff + c], weights[(size_t)n * E + e], k.limit, k);
    } else {
      const int c = j - E * ff;
      a = gated_value(row[2 * E * ff + c], row[2 * E * ff + shared + c], 1.f, k.limit_shared, k);
    }
    out[(size_t)n * total + j] = from_f32<T>(a);
  }
}

// the chosen experts alone: hs[n, k * ff + j] = act of expert chosen[n, k]'s rows j against y[n], and the shared
// expert's behind them; `up` is the stacked matrix [2 (E * ff + shared), H]
template <typename T>
__global__ void __launch_bounds__(256)
expert_rows_gated_up_kernel(const T* __restrict__ y, int H, const T* __restrict__ up, const int* __restrict__ chosen,
                            const float* __restrict__ weights, int E, int top, int ff, int shared, GateTerms kt, bool vec,
                            T* __restrict__ hs) {
  const int slots = top + (shared ? 1 : 0);
  const int n = blockIdx.x / slots, k = blockIdx.x % slots;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  int base, count;
  float scale = 1.f, limit = kt.limit_shared;
  if (k < top) {
    const int e = chosen[(size_t)n * top + k];
    base = 2 * e * ff;
    count = ff;
    scale = weights[(size_t)n * E + e];
    limit = kt.limit;
  } else {
    base = 2 * E * ff;
    count = shared;
  }
  const T* row = y + (size_t)n * H;
  T* out = hs + (size_t)n * (top * ff + shared) + (size_t)k * ff;
#pragma unroll
  for (int r = 0; r < ER_ROWS / 4; ++r) {
    const int j = blockIdx.y * ER_ROWS + wave * (ER_ROWS / 4) + r;
    if (j >= count) break;
    const float g = wave_dot(up + (size_t)(base + j) * H, row, H, vec, lane);
    const float u = wave_dot(up + (size_t)(base + count + j) * H, row, H, vec, lane);
    if (lane == 0) out[j] = from_f32<T>(gated_value(g, u, scale, limit, kt));
  }
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_route(const void* h, int dt, int n, int W, const float* wr, int E, int groups, int keep, int top, int logistic,
             float* weights, int* chosen, hipStream_t st) {
  TL_REQUIRE(n >= 0 && W > 0 && E > 0 && E <= RT_MAX_E && top > 0 && top <= E, "route: bad sizes n=%d W=%d E=%d top=%d (experts up to %d)",
             n, W, E, top, RT_MAX_E);
  TL_REQUIRE(groups >= 0 && (groups == 0 || (E % groups == 0 && keep > 0 && keep <= groups && keep * (E / groups) >= top)),
             "route: %d experts in %d groups of which %d are kept cannot give %d", E, groups, keep, top);
  TL_REQUIRE(h && wr && weights, "route: a buffer is missing");
  if (n == 0) return 0;
  const bool vec = W % 4 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)wr % 16 == 0;
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "route: unknown dtype code %d", dt);
  const bool few = n <= 64 && E > 4;             // fewer rows than compute units: more waves a row
  if (dt == DT_F32 && few)
    route_kernel<float, 1024><<<n, 1024, 0, st>>>((const float*)h, W, wr, E, groups, keep, top, logistic, weights, chosen, vec);
  else if (dt == DT_F32)
    route_kernel<float, 256><<<n, 256, 0, st>>>((const float*)h, W, wr, E, groups, keep, top, logistic, weights, chosen, vec);
  else if (few)
    route_kernel<bf16, 1024><<<n, 1024, 0, st>>>((const bf16*)h, W, wr, E, groups, keep, top, logistic, weights, chosen, vec);
  else
    route_kernel<bf16, 256><<<n, 256, 0, st>>>((const bf16*)h, W, wr, E, groups, keep, top, logistic, weights, chosen, vec);
  TL_LAUNCH_CHECK("route");
  return 0;
}

int tl_expert_act(const float* u, const float* weights, int n, int E, int ff, int total, int act, void* out, int dt,
                  hipStream_t st) {
  TL_REQUIRE(n >= 0 && E >= 0 && ff > 0 && total >= E * ff && (act == 0 || act == 1), "expert_act: bad sizes E=%d ff=%d total=%d act=%d",
             E, ff, total, act);
  TL_REQUIRE(u && out && (E == 0 || weights), "expert_act: a buffer is missing");
  if (n == 0) return 0;
  const dim3 grid(n, min((total + 255) / 256, 64));
  if (dt == DT_F32)
    expert_act_kernel<float><<<grid, 256, 0, st>>>(u, weights, E, ff, total, act, (float*)out);
  else if (dt == DT_BF16)
    expert_act_kernel<bf16><<<grid, 256, 0, st>>>(u, weights, E, ff, total, act, (bf16*)out);
  else
    TL_REQUIRE(false, "expert_act: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("expert_act");
  return 0;
}

// y [n, H], up [E * ff + shared, H], chosen int [n, top], weights [n, E] -> hs [n, top * ff + shared], all of dtype dt
int tl_expert_rows_up(const void* y, int H, const void* up, const int* chosen, const float* weights, int n, int E, int top, int ff,
                      int shared, int act, void* hs, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && E > 0 && top > 0 && top <= E && ff > 0 && shared >= 0 && (act == 0 || act == 1),
             "expert_rows_up: bad sizes H=%d E=%d top=%d ff=%d shared=%d act=%d", H, E, top, ff, shared, act);
  TL_REQUIRE(y && up && chosen && weights && hs, "expert_rows_up: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "expert_rows_up: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const int slots = top + (shared ? 1 : 0);
  const int most = ff > shared ? ff : shared;
  const dim3 grid(n * slots, (most + ER_ROWS - 1) / ER_ROWS);
  const int per = dt == DT_BF16 ? 8 : 4;
  const bool vec = H % per == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)up % 16 == 0;
  if (dt == DT_F32)
    expert_rows_up_kernel<float><<<grid, 256, 0, st>>>((const float*)y, H, (const float*)up, chosen, weights, E, top, ff, shared, act, vec,
                                                       (float*)hs);
  else
    expert_rows_up_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)y, H, (const bf16*)up, chosen, weights, E, top, ff, shared, act, vec,
                                                      (bf16*)hs);
  TL_LAUNCH_CHECK("expert_rows_up");
  return 0;
}

// hs [n, top * ff + shared], down [H, E * ff + shared] of dtype dt -> out float [n, H], added to or stored
int tl_expert_rows_down(const void* hs, const void* down, const int* chosen, int n, int E, int top, int ff, int shared, int H,
                        int accumulate, float* out, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && E > 0 && top > 0 && top <= E && ff > 0 && shared >= 0, "expert_rows_down: bad sizes H=%d E=%d top=%d ff=%d shared=%d",
             H, E, top, ff, shared);
  TL_REQUIRE(hs && down && chosen && out, "expert_rows_down: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "expert_rows_down: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const dim3 grid(n, (H + ER_ROWS - 1) / ER_ROWS);
  const int per = dt == DT_BF16 ? 8 : 4;
  const bool vec = ff % per == 0 && shared % per == 0 && (uintptr_t)hs % 16 == 0 && (uintptr_t)down % 16 == 0;
  if (dt == DT_F32)
    expert_rows_down_kernel<float><<<grid, 256, 0, st>>>((const float*)hs, (const float*)down, chosen, E, top, ff, shared, H, vec, accumulate, out);
  else
    expert_rows_down_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)hs, (const bf16*)down, chosen, E, top, ff, shared, H, vec, accumulate, out);
  TL_LAUNCH_CHECK("expert_rows_down");
  return 0;
}

// gu float [n, 2 (E * ff + shared)], weights float [n, E] (E == 0: none) -> out [n, E * ff + shared] of dtype dt
int tl_expert_gated_act(const float* gu, const float* weights, int n, int E, int ff, int shared, float limit, float limit_shared,
                        float alpha, float shift, int on_input, void* out, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && E >= 0 && ff >= 0 && shared >= 0 && E * ff + shared > 0, "expert_gated_act: bad sizes E=%d ff=%d shared=%d", E, ff, shared);
  TL_REQUIRE(gu && out && (E == 0 || weights), "expert_gated_act: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "expert_gated_act: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const int total = E * ff + shared;
  const dim3 grid(n, min((total + 255) / 256, 64));
  const GateTerms k{limit, limit_shared, alpha, shift, on_input};
  if (dt == DT_F32) expert_gated_act_kernel<float><<<grid, 256, 0, st>>>(gu, weights, E, ff, shared, k, (float*)out);
  else expert_gated_act_kernel<bf16><<<grid, 256, 0, st>>>(gu, weights, E, ff, shared, k, (bf16*)out);
  TL_LAUNCH_CHECK("expert_gated_act");
  return 0;
}

// y [n, H], up [2 (E * ff + shared), H], chosen int [n, top], weights [n, E] -> hs [n, top * ff + shared], all of dtype dt
int tl_expert_rows_gated_up(const void* y, int H, const void* up, const int* chosen, const float* weights, int n, int E, int top,
                            int ff, int shared, float limit, float limit_shared, float alpha, float shift, int on_input, void* hs,
                            int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && E > 0 && top > 0 && top <= E && ff > 0 && shared >= 0,
             "expert_rows_gated_up: bad sizes H=%d E=%d top=%d ff=%d shared=%d", H, E, top, ff, shared);
  TL_REQUIRE(y && up && chosen && weights && hs, "expert_rows_gated_up: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "expert_rows_gated_up: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const int slots = top + (shared ? 1 : 0);
  const int most = ff > shared ? ff : shared;
  const dim3 grid(n * slots, (most + ER_ROWS - 1) / ER_ROWS);
  const int per = dt == DT_BF16 ? 8 : 4;
  const bool vec = H % per == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)up % 16 == 0;
  const GateTerms k{limit, limit_shared, alpha, shift, on_input};
  if (dt == DT_F32)
    expert_rows_gated_up_kernel<float><<<grid, 256, 0, st>>>((const float*)y, H, (const float*)up, chosen, weights, E, top, ff, shared, k,
                                                             vec, (float*)hs);
  else
    expert_rows_gated_up_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)y, H, (const bf16*)up, chosen, weights, E, top, ff, shared, k,
                                                            vec, (bf16*)hs);
  TL_LAUNCH_CHECK("expert_rows_gated_up");
  return 0;
}

}  // extern "C"
