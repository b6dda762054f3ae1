// A recurrence per channel whose update gate z and candidate c are functions of the present row only:
//
//     z_t = logistic(a_t + bz) ,  c_t = cand(b_t + bx) ,  S_t = (1 - z_t) S_(t-1) + z_t c_t ,
//     out_t = S_t * silu(g_t)
//
// with cand(u) = u + 1/2 for u >= 0 and logistic(u) below (positive and continuous), and a row of
// the fused projection [a | b | g] of W channels each, in float.  S is one float a channel and
// sequence, kept in the sequence's block of the cache between steps; gates, candidates, the state
// and the output's gate are float whatever the compute type is.
//
// Two ways through a step's rows.  `rows`: a thread per (sequence, channel) goes through the
// sequence's rows in order: single tokens and short portions.  `chunks` + `apply`: a sequence's rows
// are cut into runs of RC_CHUNK; a first kernel works out, per run and channel, the product P of the
// (1 - z) and the state Q that the run reaches from zero; a second kernel folds the runs before
// its own, S_in = P_r S + Q_r in order from the sequence's state at the step's start, and goes
// through its run from there.  The recurrence is linear in S, so this is the same sum in another
// order of rounding; every run has a workgroup of its own, which is what a long prompt needs.
#include "common.hpp"

namespace tl {

constexpr int RC_CHUNK = 32;

__device__ __forceinline__ float logistic(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float candidate(float u) { return u >= 0.f ? u + 0.5f : logistic(u); }

template <typename TO>
__global__ void __launch_bounds__(256)
gru_rows_kernel(const float* __restrict__ proj, const float* __restrict__ bz, const float* __restrict__ bx, int W,
                float* __restrict__ state, long long state_stride, const int* __restrict__ cu_seqlens,
                const int* __restrict__ slots, TO* __restrict__ out) {
  const int ch = blockIdx.x * 256 + threadIdx.x;
  const int b = blockIdx.y;
  if (ch >= W) return;
  const int r0 = cu_seqlens[b], r1 = cu_seqlens[b + 1];
  float* sp = state + (long long)slots[b] * state_stride + ch;
  float S = *sp;
  const float zb = bz ? bz[ch] : 0.f, xb = bx ? bx[ch] : 0.f;
  for (int r = r0; r < r1; ++r) {
    const float* row = proj + (size_t)r * 3 * W;
    const float z = logistic(row[ch] + zb);
    const float c = candidate(row[W + ch] + xb);
    const float g = row[2 * W + ch];
    S = (1.0f - z) * S + z * c;
    out[(size_t)r * W + ch] = from_f32<TO>(S * (g * logistic(g)));
  }
  *sp = S;
}

// run `item` of the step: its sequence and its rows
__device__ __forceinline__ bool run_of(int item, const int* cu_seqlens, int B, int& b, int& first, int& r0, int& r1) {
  int t = item;
  for (b = 0; b < B; ++b) {
    const int runs = (cu_seqlens[b + 1] - cu_seqlens[b] + RC_CHUNK - 1) / RC_CHUNK;
    if (t < runs) break;
    t -= runs;
  }
  if (b == B) return false;
  first = item - t;                                  // the sequence's first run
  r0 = cu_seqlens[b] + t * RC_CHUNK;
  r1 = min(r0 + RC_CHUNK, cu_seqlens[b + 1]);
  return true;
}

__global__ void __launch_bounds__(256)
gru_chunks_kernel(const float* __restrict__ proj, const float* __restrict__ bz, const float* __restrict__ bx, int W,
                  const int* __restrict__ cu_seqlens, int B, float* __restrict__ P, float* __restrict__ Q) {
  const int ch = blockIdx.x * 256 + threadIdx.x;
  int b, first, r0, r1;
  if (ch >= W || !run_of(blockIdx.y, cu_seqlens, B, b, first, r0, r1)) return;
  const float zb = bz ? bz[ch] : 0.f, xb = bx ? bx[ch] : 0.f;
  float p = 1.f, q = 0.f;
#pragma unroll 8
  for (int r = r0; r < r1; ++r) {
    const float* row = proj + (size_t)r * 3 * W;
    const float z = logistic(row[ch] + zb);
    const float c = candidate(row[W + ch] + xb);
    p *= 1.0f - z;
    q = (1.0f - z) * q + z * c;
  }
  P[(size_t)blockIdx.y * W + ch] = p;
  Q[(size_t)blockIdx.y * W + ch] = q;
}

template <typename TO>
__global__ void __launch_bounds__(256)
gru_apply_kernel(const float* __restrict__ proj, const float* __restrict__ bz, const float* __restrict__ bx, int W,
                 const float* __restrict__ P, const float* __restrict__ Q, const float* __restrict__ start,
                 float* __restrict__ state, long long state_stride, const int* __restrict__ cu_seqlens,
                 const int* __restrict__ slots, int B, TO* __restrict__ out) {
  const int ch = blockIdx.x * 256 + threadIdx.x;
  int b, first, r0, r1;
  if (ch >= W || !run_of(blockIdx.y, cu_seqlens, B, b, first, r0, r1)) return;
  float S = start[(size_t)b * W + ch];
  for (int i = first; i < (int)blockIdx.y; ++i) S = P[(size_t)i * W + ch] * S + Q[(size_t)i * W + ch];
  const float zb = bz ? bz[ch] : 0.f, xb = bx ? bx[ch] : 0.f;
#pragma unroll 8
  for (int r = r0; r < r1; ++r) {
    const float* row = proj + (size_t)r * 3 * W;
    const float z = logistic(row[ch] + zb);
    const float c = candidate(row[W + ch] + xb);
    const float g = row[2 * W + ch];
    S = (1.0f - z) * S + z * c;
    out[(size_t)r * W + ch] = from_f32<TO>(S * (g * logistic(g)));
  }
  if (r1 == cu_seqlens[b + 1]) state[(long long)slots[b] * state_stride + ch] = S;
}

// start[b] = state[slots[b]]: the states as the step finds them, where no run writes
__global__ void __launch_bounds__(256)
gru_start_kernel(const float* __restrict__ state, long long state_stride, const int* __restrict__ slots, int W,
                 float* __restrict__ start) {
  const int ch = blockIdx.x * 256 + threadIdx.x;
  if (ch < W) start[(size_t)blockIdx.y * W + ch] = state[(long long)slots[blockIdx.y] * state_stride + ch];
}

}  // namespace tl

using namespace tl;

extern "C" {

int tl_gated_recurrence_chunk(void) { return RC_CHUNK; }

// proj float [n, 3 W] = [a | b | g]; bz, bx float [W] or null; state float [slots, >= W] with rows state_stride apart;
// out [n, W] of dtype dt.  n_runs: 0 = a thread goes through a sequence's rows in order; else the number of runs of
// RC_CHUNK rows in the step (sum over sequences of ceil(rows / RC_CHUNK)), with scratch float [(2 n_runs + B) W].
int tl_gated_recurrence(const float* proj, const float* bz, const float* bx, int n, int W, float* state,
                        long long state_stride, const int* cu_seqlens, const int* slots, int B, int n_runs, float* scratch,
                        void* out, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && W > 0 && B > 0 && n_runs >= 0 && state_stride >= W, "gated_recurrence: bad sizes n=%d W=%d B=%d runs=%d stride=%lld",
             n, W, B, n_runs, state_stride);
  TL_REQUIRE(proj && state && cu_seqlens && slots && out && (n_runs == 0 || scratch), "gated_recurrence: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "gated_recurrence: unknown dtype code %d", dt);
  TL_REQUIRE(B <= 65535 && n_runs <= 65535, "gated_recurrence: %d sequences or %d runs are too many for one launch", B, n_runs);
  if (n == 0) return 0;
  const unsigned gx = (W + 255) / 256;
  if (n_runs == 0) {
    if (dt == DT_F32) gru_rows_kernel<float><<<dim3(gx, B), 256, 0, st>>>(proj, bz, bx, W, state, state_stride, cu_seqlens, slots, (float*)out);
    else gru_rows_kernel<bf16><<<dim3(gx, B), 256, 0, st>>>(proj, bz, bx, W, state, state_stride, cu_seqlens, slots, (bf16*)out);
    TL_LAUNCH_CHECK("gated_recurrence rows");
    return 0;
  }
  float* P = scratch;
  float* Q = P + (size_t)n_runs * W;
  float* start = Q + (size_t)n_runs * W;
  gru_start_kernel<<<dim3(gx, B), 256, 0, st>>>(state, state_stride, slots, W, start);
  TL_LAUNCH_CHECK("gated_recurrence start");
  gru_chunks_kernel<<<dim3(gx, n_runs), 256, 0, st>>>(proj, bz, bx, W, cu_seqlens, B, P, Q);
  TL_LAUNCH_CHECK("gated_recurrence chunks");
  if (dt == DT_F32)
    gru_apply_kernel<float><<<dim3(gx, n_runs), 256, 0, st>>>(proj, bz, bx, W, P, Q, start, state, state_stride, cu_seqlens, slots, B, (float*)out);
  else
    gru_apply_kernel<bf16><<<dim3(gx, n_runs), 256, 0, st>>>(proj, bz, bx, W, P, Q, start, state, state_stride, cu_seqlens, slots, B, (bf16*)out);
  TL_LAUNCH_CHECK("gated_recurrence apply");
  return 0;
}

}  // extern "C"
