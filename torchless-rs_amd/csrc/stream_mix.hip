// What happens to the residual stream between the sublayers of designs that keep more than one
// version of it or norm a sublayer on both sides.
//
// depth_average: the stream that goes on after run t is a weighted sum of the results of all
// runs so far, kept[0] being the embedding's output:
//     kept[t] = x ;  x = sum_{j <= t} c[j] * kept[j]
// (float throughout; kept is [T + 1, n, H]).
//
// layernorm_add_norm: a sublayer's result z goes through a layer norm (weight and bias) into the
// stream, and the norm that reads the stream next runs on the new row in the same pass:
//     x += LN(z + bias; w1, b1) ;  out = LN(x; w2, b2)        (the second part optional)
// with LN(t; w, b) = (t - mean) / sqrt(mean((t - mean)^2) + eps) * w + b.  The row stays in
// registers: one read of z and x, one write of x and out.  Between the two the weighted sum
// above may take place on the row (`kept` given): the new x is kept as version t and replaced
// by the sum, which the second norm then reads.
#include "common.hpp"

namespace tl {

__global__ void __launch_bounds__(256)
depth_average_kernel(float* __restrict__ x, float* __restrict__ kept, const float* __restrict__ c, int t,
                     long long total, bool vec) {
  const long long i0 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i0 >= total) return;
  if (vec) {
    const float4 v = *reinterpret_cast<const float4*>(x + i0);
    *reinterpret_cast<float4*>(kept + (long long)t * total + i0) = v;
    const float ct = c[t];
    float4 a = make_float4(ct * v.x, ct * v.y, ct * v.z, ct * v.w);
    for (int j = t - 1; j >= 0; --j) {
      const float4 k = *reinterpret_cast<const float4*>(kept + (long long)j * total + i0);
      const float cj = c[j];
      a.x = fmaf(cj, k.x, a.x); a.y = fmaf(cj, k.y, a.y); a.z = fmaf(cj, k.z, a.z); a.w = fmaf(cj, k.w, a.w);
    }
    *reinterpret_cast<float4*>(x + i0) = a;
    return;
  }
  for (long long i = i0; i < total && i < i0 + 4; ++i) {
    const float v = x[i];
    kept[(long long)t * total + i] = v;
    float a = c[t] * v;
    for (int j = t - 1; j >= 0; --j) a = fmaf(c[j], kept[(long long)j * total + i], a);
    x[i] = a;
  }
}

// H % 4 == 0, H <= 1024 * IT
template <typename TO, int IT>
__global__ void __launch_bounds__(256)
layernorm_add_norm_kernel(const float* __restrict__ z, const float* __restrict__ bias, const float* __restrict__ w1,
                          const float* __restrict__ b1, float eps1, float* __restrict__ x, const float* __restrict__ w2,
                          const float* __restrict__ b2, float eps2, TO* __restrict__ out, int H, float* __restrict__ kept,
                          const float* __restrict__ coef, int t, long long total) {
  __shared__ float sh[4];
  const int n = blockIdx.x;
  const int nv = H / 4;
  const float4* zr = reinterpret_cast<const float4*>(z + (size_t)n * H);
  float4* xr = reinterpret_cast<float4*>(x + (size_t)n * H);
  float4 v[IT];
  // mean and deviations of the row in v, then the row over its deviation's root mean square
  auto normalise = [&](float eps) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i)
      if (threadIdx.x + 256 * i < nv) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    const float mean = block_sum<256>(s, sh) / (float)H;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < IT; ++i)
      if (threadIdx.x + 256 * i < nv) {
        v[i].x -= mean; v[i].y -= mean; v[i].z -= mean; v[i].w -= mean;
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
      }
    return sqrtf(block_sum<256>(ss, sh) / (float)H + eps);
  };
  auto affine = [&](float4 t, float sd, const float* w, const float* b, int c) {
    const float4 g = reinterpret_cast<const float4*>(w)[c];
    float4 y = make_float4((t.x / sd) * g.x, (t.y / sd) * g.y, (t.z / sd) * g.z, (t.w / sd) * g.w);
    if (b) {
      const float4 e = reinterpret_cast<const float4*>(b)[c];
      y.x += e.x; y.y += e.y; y.z += e.z; y.w += e.w;
    }
    return y;
  };
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      v[i] = zr[c];
      if (bias) {
        const float4 e = reinterpret_cast<const float4*>(bias)[c];
        v[i].x += e.x; v[i].y += e.y; v[i].z += e.z; v[i].w += e.w;
      }
    }
  }
  const float sd1 = normalise(eps1);
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      const float4 y = affine(v[i], sd1, w1, b1, c);
      float4 a = xr[c];
      a.x += y.x; a.y += y.y; a.z += y.z; a.w += y.w;
      if (kept != nullptr) {                    // version t of the stream, and the weighted sum of versions 0 .. t
        const long long at = (long long)n * H + 4 * c;
        *reinterpret_cast<float4*>(kept + (long long)t * total + at) = a;
        const float ct = coef[t];
        a.x *= ct; a.y *= ct; a.z *= ct; a.w *= ct;
        for (int j = t - 1; j >= 0; --j) {
          const float4 k = *reinterpret_cast<const float4*>(kept + (long long)j * total + at);
          const float cj = coef[j];
          a.x = fmaf(cj, k.x, a.x); a.y = fmaf(cj, k.y, a.y); a.z = fmaf(cj, k.z, a.z); a.w = fmaf(cj, k.w, a.w);
        }
      }
      xr[c] = a;
      v[i] = a;
    }
  }
  if (w2 == nullptr) return;
  const float sd2 = normalise(eps2);
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      const float4 y = affine(v[i], sd2, w2, b2, c);
      TO* o = out + (size_t)n * H + 4 * c;
      o[0] = from_f32<TO>(y.x); o[1] = from_f32<TO>(y.y); o[2] = from_f32<TO>(y.z); o[3] = from_f32<TO>(y.w);
    }
  }
}

}  // namespace tl

using namespace tl;

extern "C" {

// x float [n * H] (total), kept float [>= (t + 1) * total], c float [>= t + 1]
int tl_depth_average(float* x, float* kept, const float* c, int t, long long total, hipStream_t st) {
  TL_REQUIRE(t >= 0 && total >= 0, "depth_average: bad sizes t=%d total=%lld", t, total);
  TL_REQUIRE(x && kept && c, "depth_average: a buffer is missing");
  if (total == 0) return 0;
  const bool vec = total % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)kept % 16 == 0;
  const long long blocks = (total + 1023) / 1024;
  TL_REQUIRE(blocks < 2147483000LL, "depth_average: %lld values are too many for one launch", total);
  depth_average_kernel<<<(unsigned)blocks, 256, 0, st>>>(x, kept, c, t, total, vec);
  TL_LAUNCH_CHECK("depth_average");
  return 0;
}

// x += LN(z + bias; w1, b1); with kept: kept[t] = x, x = sum_{j <= t} coef[j] kept[j] (kept float [> t, n, H]); with w2:
// out = LN(x; w2, b2).  Rows of a multiple of 4 up to 8,192 channels, 16-byte aligned (the caller takes the steps one
// by one for any other).
int tl_layernorm_add_norm(const float* z, const float* bias, const float* w1, const float* b1, float eps1, float* x,
                          const float* w2, const float* b2, float eps2, void* out, int out_dt, int n, int H, float* kept,
                          const float* coef, int t, hipStream_t st) {
  TL_REQUIRE(kept == nullptr || (coef != nullptr && t >= 0 && (uintptr_t)kept % 16 == 0), "layernorm_add_norm: versions of the stream without weights");
  const long long total = (long long)n * H;
  TL_REQUIRE(n >= 0 && H > 0, "layernorm_add_norm: bad sizes n=%d H=%d", n, H);
  TL_REQUIRE(z && w1 && x && (w2 == nullptr || out != nullptr), "layernorm_add_norm: a buffer is missing");
  TL_REQUIRE(out_dt == DT_F32 || out_dt == DT_BF16, "layernorm_add_norm: unknown dtype code %d", out_dt);
  const bool al = (uintptr_t)z % 16 == 0 && (uintptr_t)bias % 16 == 0 && (uintptr_t)w1 % 16 == 0 && (uintptr_t)b1 % 16 == 0 &&
                  (uintptr_t)x % 16 == 0 && (uintptr_t)w2 % 16 == 0 && (uintptr_t)b2 % 16 == 0;
  TL_REQUIRE(H % 4 == 0 && H <= 8192 && al, "layernorm_add_norm: rows of %d channels (a multiple of 4 up to 8192, aligned)", H);
  if (n == 0) return 0;
  const bool f32 = out_dt == DT_F32;
#define TL_LAN(IT)                                                                                                          \
  do {                                                                                                                      \
    if (f32) layernorm_add_norm_kernel<float, IT><<<n, 256, 0, st>>>(z, bias, w1, b1, eps1, x, w2, b2, eps2, (float*)out, H, kept, coef, t, total); \
    else layernorm_add_norm_kernel<bf16, IT><<<n, 256, 0, st>>>(z, bias, w1, b1, eps1, x, w2, b2, eps2, (bf16*)out, H, kept, coef, t, total);       \
  } while (0)
  if (H <= 1024) TL_LAN(1);
  else if (H <= 2048) TL_LAN(2);
  else if (H <= 4096) TL_LAN(4);
  else TL_LAN(8);
#undef TL_LAN
  TL_LAUNCH_CHECK("layernorm_add_norm");
  return 0;
}

}  // extern "C"
