// A routed mixture of small feed-forward layers ("experts").
//
// Router, per row, in float: z = W_r h, s = softmax(z) over all E experts.  The experts form
// `groups` equal groups of neighbours; a group's score is its largest s, and only experts of the
// `keep` best groups can be chosen (groups == 0: every expert can).  Of those the `top` with the
// largest s are chosen; their weights are their s, not renormalised.  Of equal scores the one
// with the smaller index goes first.
//
// `route` leaves the weights as a row of E floats, zero for an expert that was not chosen.
// The experts run as ONE wide feed-forward: the rows of all up projections stacked (the shared
// expert's behind them), the activation times the row's weight of the column's expert
// (`expert_act`), and all down projections side by side: an expert with weight zero adds nothing.
#include "common.hpp"

namespace tl {

constexpr int RT_MAX_E = 1024;

template <typename T>
__global__ void __launch_bounds__(256)
route_kernel(const T* __restrict__ h, int W, const float* __restrict__ wr, int E, int groups, int keep, int top,
             float* __restrict__ weights, int* __restrict__ chosen) {
  __shared__ float s_s[RT_MAX_E];
  __shared__ float g_s[RT_MAX_E];
  __shared__ unsigned char ok_s[RT_MAX_E];
  __shared__ float sh[4];
  const int n = blockIdx.x;
  const int t = threadIdx.x, lane = t % WAVE, wave = t / WAVE;
  const T* row = h + (size_t)n * W;
  for (int e = wave; e < E; e += 4) {
    const float* w = wr + (size_t)e * W;
    float dot = 0.f;
    for (int c = lane; c < W; c += WAVE) dot = fmaf(w[c], to_f32(row[c]), dot);
    dot = wave_sum(dot);
    if (lane == 0) s_s[e] = dot;
  }
  __syncthreads();
  float m = -INFINITY;
  for (int e = t; e < E; e += 256) m = fmaxf(m, s_s[e]);
  m = block_max<256>(m, sh);
  float sum = 0.f;
  for (int e = t; e < E; e += 256) sum += expf(s_s[e] - m);
  sum = block_sum<256>(sum, sh);
  __syncthreads();
  for (int e = t; e < E; e += 256) s_s[e] = expf(s_s[e] - m) / sum;
  __syncthreads();
  if (groups > 0) {
    const int per = E / groups;
    for (int g = t; g < groups; g += 256) {
      float best = s_s[g * per];
      for (int i = 1; i < per; ++i) best = fmaxf(best, s_s[g * per + i]);
      g_s[g] = best;
    }
    __syncthreads();
    for (int g = t; g < groups; g += 256) {
      int ahead = 0;
      const float mine = g_s[g];
      for (int o = 0; o < groups; ++o) ahead += (g_s[o] > mine || (g_s[o] == mine && o < g)) ? 1 : 0;
      for (int i = 0; i < per; ++i) ok_s[g * per + i] = ahead < keep;
    }
  } else {
    for (int e = t; e < E; e += 256) ok_s[e] = 1;
  }
  __syncthreads();
  for (int e = t; e < E; e += 256) {
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

}  // namespace tl

using namespace tl;

extern "C" {

int tl_route(const void* h, int dt, int n, int W, const float* wr, int E, int groups, int keep, int top, float* weights,
             int* chosen, hipStream_t st) {
  TL_REQUIRE(n >= 0 && W > 0 && E > 0 && E <= RT_MAX_E && top > 0 && top <= E, "route: bad sizes n=%d W=%d E=%d top=%d (experts up to %d)",
             n, W, E, top, RT_MAX_E);
  TL_REQUIRE(groups >= 0 && (groups == 0 || (E % groups == 0 && keep > 0 && keep <= groups && keep * (E / groups) >= top)),
             "route: %d experts in %d groups of which %d are kept cannot give %d", E, groups, keep, top);
  TL_REQUIRE(h && wr && weights, "route: a buffer is missing");
  if (n == 0) return 0;
  if (dt == DT_F32)
    route_kernel<float><<<n, 256, 0, st>>>((const float*)h, W, wr, E, groups, keep, top, weights, chosen);
  else if (dt == DT_BF16)
    route_kernel<bf16><<<n, 256, 0, st>>>((const bf16*)h, W, wr, E, groups, keep, top, weights, chosen);
  else
    TL_REQUIRE(false, "route: unknown dtype code %d", dt);
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

}  // extern "C"
