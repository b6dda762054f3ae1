// A state-space mixer: a linear recurrence per head over a matrix state, with a short
// causal convolution before it and a gated, grouped norm behind it.
//
// A row of the input projection is [z (inner) | u (C = inner + 2*G*N) | dt (heads)] in float,
// inner = heads * dv.  u passes a convolution per channel over its last `taps` rows (zeros before
// the start of a sequence) and silu, and is then read as [x (heads*dv) | B (G*N) | C (G*N)].  With
// dt' = softplus(dt + dt_bias[h]) and a = exp(-exp(A_log[h]) * dt'), head h (which reads B and C
// of group h / (heads / G)) keeps a state S [N, dv]:
//
//   S <- a S + dt' B x^T ;   y = S^T C + D[h] x
//
// and the row's result is rms_parts(y * silu(z)) * w: the gated y cut into equal parts, each
// divided by its own root mean square (eps inside the root).  dt', a, the state and the sums
// are float whatever the storage type is; the state lives in a block per sequence,
// [conv: (taps-1) rows of C channels, the oldest first | S^T: heads * dv * N], and is carried
// from step to step.
#include "common.hpp"

namespace tl {

constexpr int SSM_MAX_TAPS = 8;
constexpr int SSM_MAX_N = 256;
constexpr int SSM_MAX_DV = 256;
constexpr int SSM_TB = 8;              // rows of a sequence that the recurrence stages at a time

__device__ __forceinline__ float silu_f(float a) { return a / (1.0f + expf(-a)); }
__device__ __forceinline__ float softplus_f(float a) { return fmaxf(a, 0.f) + log1pf(expf(-fabsf(a))); }

// out[n, c] = silu(bias[c] + sum_j w[c, j] * u[row - (taps-1-j), c]); rows before the step come
// from the sequence's block, rows before the sequence are zeros (the block is zero then).
template <typename T>
__global__ void __launch_bounds__(256)
ssm_conv_kernel(const float* __restrict__ proj, int width, int off, int C, const float* __restrict__ w,
                const float* __restrict__ bias, int taps, const float* __restrict__ conv_state, long long stride,
                const int* __restrict__ row_seq, const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
                T* __restrict__ out) {
  const int n = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = row_seq[n];
  const int i = n - cu_seqlens[b];
  const float* old = conv_state + (long long)slots[b] * stride;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    const int src = i - back;
    const float u = src >= 0 ? proj[(size_t)(n - back) * width + off + c] : old[(size_t)(taps - 1 + src) * C + c];
    acc = fmaf(w[(size_t)c * taps + j], u, acc);
  }
  out[(size_t)n * C + c] = from_f32<T>(silu_f(acc));
}

// The block's last taps-1 inputs after the step: from the step's rows, or shifted within the block.
__global__ void __launch_bounds__(256)
ssm_conv_carry_kernel(const float* __restrict__ proj, int width, int off, int C, int taps, float* __restrict__ conv_state,
                      long long stride, const int* __restrict__ cu_seqlens, const int* __restrict__ slots) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int row0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - row0;
  float* st = conv_state + (long long)slots[b] * stride;
  float old[SSM_MAX_TAPS - 1];
#pragma unroll
  for (int s = 0; s < SSM_MAX_TAPS - 1; ++s) old[s] = s < taps - 1 ? st[(size_t)s * C + c] : 0.f;
#pragma unroll
  for (int s = 0; s < SSM_MAX_TAPS - 1; ++s) {
    if (s >= taps - 1) break;
    const int src = n_new - (taps - 1) + s;
    float val = 0.f;
    if (src >= 0) {
      val = proj[(size_t)(row0 + src) * width + off + c];
    } else {
#pragma unroll
      for (int q = 0; q < SSM_MAX_TAPS - 1; ++q)
        if (q == s + n_new) val = old[q];
    }
    st[(size_t)s * C + c] = val;
  }
}

// One row a sequence: the convolution and the block's shift in one pass (a thread reads and writes its own
// channel of its own sequence alone).
template <typename T>
__global__ void __launch_bounds__(256)
ssm_conv_single_kernel(const float* __restrict__ proj, int width, int off, int C, const float* __restrict__ w,
                       const float* __restrict__ bias, int taps, float* __restrict__ conv_state, long long stride,
                       const int* __restrict__ slots, T* __restrict__ out) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  float* st = conv_state + (long long)slots[b] * stride;
  const float cur = proj[(size_t)b * width + off + c];
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps - 1; ++j) {
    const float old = st[(size_t)j * C + c];
    acc = fmaf(w[(size_t)c * taps + j], old, acc);
    if (j > 0) st[(size_t)(j - 1) * C + c] = old;
  }
  acc = fmaf(w[(size_t)c * taps + taps - 1], cur, acc);
  if (taps > 1) st[(size_t)(taps - 2) * C + c] = cur;
  out[(size_t)b * C + c] = from_f32<T>(silu_f(acc));
}

// The recurrence, row after row: one workgroup per (head, sequence, part of the head's columns).  A head's state
// is kept column by column, S^T [dv, N].  The workgroup takes `dvb` columns in groups of DC; `nsl` neighbouring
// lanes (a power of two, at most a wave) share a group: lane s keeps rows s, s + nsl, ... (R at most) of the
// group's DC columns in registers, so that a row's B and C are read once for DC columns.  The rows' x, B, C, dt'
// and decay are staged SSM_TB rows at a time; a row of the sequence costs no barrier and no exchange between
// lanes: the lanes' shares of a column's sum are left in LDS and added once a batch.
template <typename T, int R, int DC>
__global__ void __launch_bounds__(256)
ssm_scan_kernel(const T* __restrict__ u, int C, int inner, int G, int N, int heads, int dv, int dvb, int nsl, int NP,
                const float* __restrict__ proj, int width, int dt_off, const float* __restrict__ dt_bias,
                const float* __restrict__ A_log, const float* __restrict__ Dw, float* __restrict__ state, long long stride,
                const int* __restrict__ cu_seqlens, const int* __restrict__ slots, float* __restrict__ y) {
  extern __shared__ __attribute__((aligned(16))) float ssm_lds[];
  float* xs = ssm_lds;                 // [SSM_TB][dvb]
  float* Bs = xs + SSM_TB * dvb;       // [SSM_TB][NP]: NP = R * nsl >= N, zeros behind the N rows, so that the
  float* Cs = Bs + SSM_TB * NP;        // [SSM_TB][NP]  rows' loop reads without asking where N ends
  float* as = Cs + SSM_TB * NP;        // [SSM_TB]
  float* dts = as + SSM_TB;            // [SSM_TB]
  float* part = dts + SSM_TB;          // [SSM_TB][dvb][nsl]: every lane's share of a row's sums
  const int h = blockIdx.x, b = blockIdx.y, d0 = blockIdx.z * dvb;
  const int g = h / (heads / G);
  const int t = threadIdx.x;
  const int s = t % nsl, cg = t / nsl;
  const bool active = cg * DC < dvb;
  const int c0 = active ? cg * DC : 0;                // this lane's first column among the workgroup's
  const int PW = dvb * nsl;
  const int row0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - row0;
  float* S_g = state + (long long)slots[b] * stride + (size_t)h * N * dv + (size_t)(d0 + c0) * N;
  float S[R][DC];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int nr = s + r * nsl;
#pragma unroll
    for (int c = 0; c < DC; ++c) S[r][c] = (active && nr < N) ? S_g[(size_t)c * N + nr] : 0.f;
  }
  const float neg_rate = -expf(A_log[h]);
  const float bias = dt_bias[h], skip = Dw[h];
  // a batch's rows come from memory into registers while the batch before is worked on; which row and column of a
  // batch a thread fetches is the same for every batch and is worked out once (divisions by sizes that the
  // compiler does not know)
  constexpr int XE = SSM_TB * (DC == 1 ? SSM_MAX_DV : 64) / 256, BE = SSM_TB * SSM_MAX_N / 256;
  int xrow[XE], xcol[XE], brow[BE], boff[BE], blds[BE];
#pragma unroll
  for (int k = 0; k < XE; ++k) {
    const int e = t + 256 * k;
    xrow[k] = e / dvb;
    xcol[k] = e % dvb;
  }
#pragma unroll
  for (int k = 0; k < BE; ++k) {
    const int e = t + 256 * k;
    brow[k] = e / N;
    boff[k] = brow[k] * C + inner + g * N + e % N;
    blds[k] = brow[k] * NP + e % N;
  }
  float xr[XE], br[BE], cr[BE], dtr = 0.f;
  auto load = [&](int i0) {
    const int tb = min(SSM_TB, n_new - i0);
    const T* rows = u + (size_t)(row0 + i0) * C;
#pragma unroll
    for (int k = 0; k < XE; ++k) xr[k] = xrow[k] < tb ? to_f32(rows[(size_t)xrow[k] * C + h * dv + d0 + xcol[k]]) : 0.f;
#pragma unroll
    for (int k = 0; k < BE; ++k) {
      br[k] = cr[k] = 0.f;
      if (brow[k] < tb) {
        br[k] = to_f32(rows[boff[k]]);
        cr[k] = to_f32(rows[boff[k] + G * N]);
      }
    }
    if (t < tb) dtr = proj[(size_t)(row0 + i0 + t) * width + dt_off + h];
  };
  for (int e = t; e < 2 * SSM_TB * NP; e += 256) Bs[e] = 0.f;      // (Bs and Cs lie one behind the other)
  if (n_new > 0) load(0);
  for (int i0 = 0; i0 < n_new; i0 += SSM_TB) {
    const int tb = min(SSM_TB, n_new - i0);
    __syncthreads();                     // the last batch's rows and shares have been read
#pragma unroll
    for (int k = 0; k < XE; ++k)
      if (xrow[k] < tb) xs[t + 256 * k] = xr[k];
#pragma unroll
    for (int k = 0; k < BE; ++k)
      if (brow[k] < tb) {
        Bs[blds[k]] = br[k];
        Cs[blds[k]] = cr[k];
      }
    if (t < tb) {
      const float dt = softplus_f(dtr + bias);
      dts[t] = dt;
      as[t] = expf(neg_rate * dt);
    }
    __syncthreads();
    if (i0 + SSM_TB < n_new) load(i0 + SSM_TB);
#pragma unroll 2
    for (int i = 0; i < tb; ++i) {
      const float a = as[i], dt = dts[i];
      float dtx[DC], acc[DC];
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        dtx[c] = dt * xs[i * dvb + c0 + c];
        acc[c] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float Bv = Bs[i * NP + s + r * nsl], Cv = Cs[i * NP + s + r * nsl];
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          S[r][c] = fmaf(a, S[r][c], Bv * dtx[c]);
          acc[c] = fmaf(S[r][c], Cv, acc[c]);
        }
      }
      if (active) {
#pragma unroll
        for (int c = 0; c < DC; ++c) part[i * PW + (c0 + c) * nsl + s] = acc[c];
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < XE; ++k) {
      if (xrow[k] >= tb) break;
      const int i = xrow[k], c = xcol[k];
      const float* shares = part + i * PW + c * nsl;
      // (turned by c: neighbours in other banks; eight sums at a time: a load does not wait for the one before)
      float sum = 0.f;
      if (nsl >= 8) {
        float p[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int q = 0; q < nsl; q += 8) {
#pragma unroll
          for (int j = 0; j < 8; ++j) p[j] += shares[(q + j + c) & (nsl - 1)];
        }
        sum = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
      } else {
        for (int q = 0; q < nsl; ++q) sum += shares[(q + c) & (nsl - 1)];
      }
      y[(size_t)(row0 + i0 + i) * inner + h * dv + d0 + c] = fmaf(skip, xs[i * dvb + c], sum);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int nr = s + r * nsl;
#pragma unroll
    for (int c = 0; c < DC; ++c)
      if (active && nr < N) S_g[(size_t)c * N + nr] = S[r][c];
  }
}

// out[n, part] = rms(y * silu(z)) * w over each of `parts` equal parts of the row.
template <typename T>
__global__ void __launch_bounds__(256)
ssm_gate_norm_kernel(const float* __restrict__ y, const float* __restrict__ proj, int width, int inner, int parts,
                     const float* __restrict__ w, float eps, T* __restrict__ out) {
  __shared__ float sh[4];
  const int n = blockIdx.x, part = blockIdx.y;
  const int P = inner / parts;
  const float* yr = y + (size_t)n * inner + part * P;
  const float* zr = proj + (size_t)n * width + part * P;
  float ss = 0.f;
  for (int i = threadIdx.x; i < P; i += 256) {
    const float a = yr[i] * silu_f(zr[i]);
    ss += a * a;
  }
  ss = block_sum<256>(ss, sh);
  const float f = 1.0f / sqrtf(ss / (float)P + eps);
  for (int i = threadIdx.x; i < P; i += 256) {
    const float a = yr[i] * silu_f(zr[i]);
    out[(size_t)n * inner + part * P + i] = from_f32<T>(a * f * w[part * P + i]);
  }
}

}  // namespace tl

using namespace tl;

// How a head's dv columns are cut over workgroups and a workgroup's 256 lanes over its columns: lanes take DC = 4
// columns each where dv allows it, a workgroup the largest part of dv of at most `most` columns (a multiple of DC).
struct ScanShape {
  int DC, dvb, nsl, R;
};
static ScanShape scan_shape_for(int N, int dv, int DC, int most) {
  ScanShape z{DC, dv, 1, 0};
  for (int c = most; c >= DC; c -= DC)
    if (c % DC == 0 && dv % c == 0) {
      z.dvb = c;
      break;
    }
  const int groups = z.dvb / DC;
  while (z.nsl * 2 <= WAVE && z.nsl * 2 * groups <= 256 && z.nsl < N) z.nsl *= 2;
  z.R = (N + z.nsl - 1) / z.nsl;
  return z;
}
// `units`: heads x sequences.  Few of them take fewer columns a workgroup (down to 16), so that the device's
// compute units all have work; many take up to 64, so that a row's B and C are staged for more columns at once.
static ScanShape scan_shape(int N, int dv, int units) {
  if (dv % 4 == 0) {
    ScanShape best{};
    for (int most = 64; most >= 16; most /= 2) {
      const ScanShape z = scan_shape_for(N, dv, 4, most);
      if (z.R > 16) continue;
      best = z;
      if ((long long)units * (dv / z.dvb) >= 512) break;
    }
    if (best.DC == 4) return best;
  }
  return scan_shape_for(N, dv, 1, 64);
}

template <typename T>
static int scan_launch(const ScanShape& z, dim3 grid, size_t lds, hipStream_t st, const T* u, int C, int inner, int G, int N,
                       int heads, int dv, const float* proj, int width, int dt_off, const float* dt_bias, const float* A_log,
                       const float* D, float* state, long long stride, const int* cu, const int* slots, float* y) {
#define TL_SCAN(RR, DD)                                                                                                      \
  ssm_scan_kernel<T, RR, DD><<<grid, 256, lds, st>>>(u, C, inner, G, N, heads, dv, z.dvb, z.nsl, RR * z.nsl, proj, width, dt_off, dt_bias, \
                                                     A_log, D, state, stride, cu, slots, y)
  if (z.DC == 4) {
    if (z.R <= 1) TL_SCAN(1, 4);
    else if (z.R <= 2) TL_SCAN(2, 4);
    else if (z.R <= 4) TL_SCAN(4, 4);
    else if (z.R <= 8) TL_SCAN(8, 4);
    else TL_SCAN(16, 4);
  } else {
    if (z.R <= 4) TL_SCAN(4, 1);
    else if (z.R <= 8) TL_SCAN(8, 1);
    else if (z.R <= 16) TL_SCAN(16, 1);
    else if (z.R <= 32) TL_SCAN(32, 1);
    else TL_SCAN(64, 1);
  }
#undef TL_SCAN
  return 0;
}

extern "C" {

// proj [n, width]: the convolution's input are its columns off .. off + C - 1.
int tl_ssm_conv(const float* proj, int width, int off, int C, const float* w, const float* bias, int taps,
                float* conv_state, long long stride, const int* row_seq, const int* cu_seqlens, const int* slots, int n,
                int B, int single, void* out, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && B >= 0 && C > 0 && off >= 0 && off + C <= width, "ssm_conv: bad sizes n=%d C=%d off=%d width=%d", n, C,
             off, width);
  TL_REQUIRE(taps >= 1 && taps <= SSM_MAX_TAPS, "ssm_conv: %d taps (1..%d)", taps, SSM_MAX_TAPS);
  TL_REQUIRE(proj && w && conv_state && row_seq && cu_seqlens && slots && out, "ssm_conv: a buffer is missing");
  TL_REQUIRE(stride >= (long long)(taps - 1) * C, "ssm_conv: a sequence's block is too small for %d rows of %d", taps - 1, C);
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "ssm_conv: unknown dtype code %d", dt);
  if (n == 0 || B == 0) return 0;
  TL_REQUIRE(!single || n == B, "ssm_conv: %d rows of %d sequences are not one row each", n, B);
  if (single) {        // one row a sequence (row b is sequence b's): the block is shifted in the same pass
    const dim3 grid1(B, (C + 255) / 256);
    if (dt == DT_F32)
      ssm_conv_single_kernel<float><<<grid1, 256, 0, st>>>(proj, width, off, C, w, bias, taps, conv_state, stride, slots, (float*)out);
    else
      ssm_conv_single_kernel<bf16><<<grid1, 256, 0, st>>>(proj, width, off, C, w, bias, taps, conv_state, stride, slots, (bf16*)out);
    TL_LAUNCH_CHECK("ssm_conv_single");
    return 0;
  }
  const dim3 grid(n, (C + 255) / 256);
  if (dt == DT_F32)
    ssm_conv_kernel<float><<<grid, 256, 0, st>>>(proj, width, off, C, w, bias, taps, conv_state, stride, row_seq, cu_seqlens,
                                                 slots, (float*)out);
  else
    ssm_conv_kernel<bf16><<<grid, 256, 0, st>>>(proj, width, off, C, w, bias, taps, conv_state, stride, row_seq, cu_seqlens,
                                                slots, (bf16*)out);
  TL_LAUNCH_CHECK("ssm_conv");
  if (taps > 1) {
    ssm_conv_carry_kernel<<<dim3(B, (C + 255) / 256), 256, 0, st>>>(proj, width, off, C, taps, conv_state, stride, cu_seqlens,
                                                                     slots);
    TL_LAUNCH_CHECK("ssm_conv_carry");
  }
  return 0;
}

// u [n, C] = [x | B | C] after the convolution; proj [n, width] holds dt at column dt_off + h.
int tl_ssm_scan(const void* u, int dt, int C, int G, int N, int heads, int dv, const float* proj, int width, int dt_off,
                const float* dt_bias, const float* A_log, const float* D, float* state, long long stride,
                const int* cu_seqlens, const int* slots, int n, int B, float* y, hipStream_t st) {
  TL_REQUIRE(n >= 0 && B >= 0 && heads > 0 && G > 0 && heads % G == 0 && N > 0 && dv > 0, "ssm_scan: bad sizes heads=%d G=%d N=%d dv=%d",
             heads, G, N, dv);
  TL_REQUIRE(N <= SSM_MAX_N && dv <= SSM_MAX_DV, "ssm_scan: a state of %d x %d is not served (up to %d x %d)", N, dv, SSM_MAX_N,
             SSM_MAX_DV);
  const int inner = heads * dv;
  TL_REQUIRE(C == inner + 2 * G * N && dt_off >= 0 && dt_off + heads <= width, "ssm_scan: %d channels for heads=%d dv=%d G=%d N=%d", C,
             heads, dv, G, N);
  const ScanShape z = scan_shape(N, dv, heads * B);
  TL_REQUIRE(z.R <= 64, "ssm_scan: a state of %d x %d gives a thread %d rows (at most 64)", N, dv, z.R);
  TL_REQUIRE(stride >= (long long)heads * N * dv, "ssm_scan: a sequence's block is too small");
  TL_REQUIRE(u && proj && dt_bias && A_log && D && state && cu_seqlens && slots && y, "ssm_scan: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "ssm_scan: unknown dtype code %d", dt);
  if (n == 0 || B == 0) return 0;
  const dim3 grid(heads, B, dv / z.dvb);
  int Rt = z.DC == 4 ? 1 : 4;                          // the rows of the kernel that `scan_launch` picks
  while (Rt < z.R) Rt *= 2;
  const size_t lds = sizeof(float) * ((size_t)SSM_TB * (z.dvb + 2 * Rt * z.nsl) + 2 * SSM_TB + (size_t)SSM_TB * z.dvb * z.nsl);
  if (dt == DT_F32)
    scan_launch<float>(z, grid, lds, st, (const float*)u, C, inner, G, N, heads, dv, proj, width, dt_off, dt_bias, A_log, D, state, stride,
                       cu_seqlens, slots, y);
  else
    scan_launch<bf16>(z, grid, lds, st, (const bf16*)u, C, inner, G, N, heads, dv, proj, width, dt_off, dt_bias, A_log, D, state, stride,
                      cu_seqlens, slots, y);
  TL_LAUNCH_CHECK("ssm_scan");
  return 0;
}

// y [n, inner] float, z = the first `inner` columns of proj [n, width].
int tl_ssm_gate_norm(const float* y, const float* proj, int width, int inner, int parts, const float* w, float eps, int n,
                     void* out, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && inner > 0 && parts > 0 && inner % parts == 0 && inner <= width, "ssm_gate_norm: bad sizes inner=%d parts=%d width=%d",
             inner, parts, width);
  TL_REQUIRE(y && proj && w && out, "ssm_gate_norm: a buffer is missing");
  TL_REQUIRE(dt == DT_F32 || dt == DT_BF16, "ssm_gate_norm: unknown dtype code %d", dt);
  if (n == 0) return 0;
  const dim3 grid(n, parts);
  if (dt == DT_F32)
    ssm_gate_norm_kernel<float><<<grid, 256, 0, st>>>(y, proj, width, inner, parts, w, eps, (float*)out);
  else
    ssm_gate_norm_kernel<bf16><<<grid, 256, 0, st>>>(y, proj, width, inner, parts, w, eps, (bf16*)out);
  TL_LAUNCH_CHECK("ssm_gate_norm");
  return 0;
}

}  // extern "C"
