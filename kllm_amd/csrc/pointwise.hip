// Per-token steps around the products of layers that are not Llama's: additive sinusoidal
// positions, an activation without a gate (with learned constants), and the norm of a layer
// whose sub-layers run side by side: it adds a scaled sum of up to two sub-layers' outputs
// and a bias to the residual stream and normalises the result in groups of channels.
// Everything here is computed in 32-bit.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

// x[t][2i] += sin(angle), x[t][2i + 1] += cos(angle), angle = p * base^(-2i / d) in double; a thread
// takes one angle.
__global__ void add_sinusoid_kernel(float* __restrict__ x, const int* __restrict__ positions, int n, int d,
                                    double log_base) {
  const int pairs = (d + 1) / 2;
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long)n * pairs) return;
  const int t = (int)(idx / pairs), i = (int)(idx % pairs);
  const double angle = (double)positions[t] * exp(-(2.0 * i / (double)d) * log_base);
  double sn, cs;
  sincos(angle, &sn, &cs);
  float* row = x + (long)t * d;
  row[2 * i] += (float)sn;
  if (2 * i + 1 < d) row[2 * i + 1] += (float)cs;
}

template <typename TOUT>
__global__ void unary_act_kernel(const float* __restrict__ in, int nsplit, long split_stride, int in_row_stride,
                                 int f, TOUT* __restrict__ out, long count, int act,
                                 const float* __restrict__ params) {
  const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const long src = in_row_stride == f ? idx : (idx / f) * in_row_stride + idx % f;
  float a_pos = 0.f, a_neg = 0.f;
  if (act == ACT_XIELU) {
    a_pos = softplus_f32(params[0]);
    a_neg = softplus_f32(params[1]);
  }
  float z = 0.f;
  for (int s = 0; s < nsplit; ++s) z += in[src + s * split_stride];
  out[idx] = from_f32<TOUT>(unary_act(z, act, a_pos, a_neg));
}

constexpr int kGroupNormThreads = 256;

// One workgroup per row.  v = x[src] + mult * (sum of d1's slices + sum of d2's slices + bias);
// x[src] = v when write_x; out[r] = v / sqrt(mean over the channel's group of v^2 + eps) * w.
// A group's sum of squares is taken by one wave over a fixed cut of the group, in a fixed
// order, so a row's result does not depend on what else the launch holds.
template <typename TOUT>
__global__ __launch_bounds__(kGroupNormThreads) void group_norm_add_kernel(
    float* __restrict__ x, const float* __restrict__ d1, int ns1, long st1, const float* __restrict__ d2, int ns2,
    long st2, const float* __restrict__ bias, float mult, const float* __restrict__ w, TOUT* __restrict__ out,
    const int* __restrict__ rows, int d, int groups, int segs, float eps, int write_x) {
  extern __shared__ float v_lds[];          // [d] the row, then [groups * segs] partial sums
  float* part = v_lds + d;
  const long r = blockIdx.x;
  const long src = rows ? rows[r] : r;
  float* xr = x + src * d;
  const int tid = threadIdx.x;
  const bool adds = d1 || d2 || bias;
  for (int i = tid; i < d; i += kGroupNormThreads) {
    float v = xr[i];
    if (adds) {
      float s = 0.f;
      if (d1)
        for (int k = 0; k < ns1; ++k) s += d1[src * d + i + k * st1];
      if (d2)
        for (int k = 0; k < ns2; ++k) s += d2[src * d + i + k * st2];
      if (bias) s += bias[i];
      v = fmaf(mult, s, v);
      if (write_x) xr[i] = v;
    }
    v_lds[i] = v;
  }
  if (!out) return;
  __syncthreads();
  const int lane = tid % kWave, wave = tid / kWave, nwaves = kGroupNormThreads / kWave;
  const int gsz = d / groups;
  const int seg_len = (gsz + segs - 1) / segs;
  for (int u = wave; u < groups * segs; u += nwaves) {
    const int g = u / segs, sg = u % segs;
    const int lo = g * gsz + sg * seg_len, hi = min(g * gsz + gsz, lo + seg_len);
    float ss = 0.f;
    for (int i = lo + lane; i < hi; i += kWave) ss = fmaf(v_lds[i], v_lds[i], ss);
    ss = wave_sum(ss);
    if (lane == 0) part[u] = ss;
  }
  __syncthreads();
  for (int i = tid; i < d; i += kGroupNormThreads) {
    const int g = i / gsz;
    float ss = 0.f;
    for (int sg = 0; sg < segs; ++sg) ss += part[g * segs + sg];
    const float rstd = 1.f / sqrtf(ss / (float)gsz + eps);
    out[r * d + i] = from_f32<TOUT>(v_lds[i] * rstd * w[i]);
  }
}

// The same for rows of up to 4 * 256 * KEEP channels in groups that are multiples of four
// channels: a thread keeps its channels in registers, four at a time, and every load is 16 bytes.
constexpr int kGroupNormMaxGroups = 8;

template <typename TOUT, int KEEP>
__global__ __launch_bounds__(kGroupNormThreads) void group_norm_add_vec_kernel(
    float* __restrict__ x, const float* __restrict__ d1, int ns1, long st1, const float* __restrict__ d2, int ns2,
    long st2, const float* __restrict__ bias, float mult, const float* __restrict__ w, TOUT* __restrict__ out,
    const int* __restrict__ rows, int d, int groups, float eps, int write_x) {
  __shared__ float red[16];
  __shared__ float rstd_g[kGroupNormMaxGroups];
  const long r = blockIdx.x;
  const long src = rows ? rows[r] : r;
  const int tid = threadIdx.x, chunks = d / 4;
  floatx4* xr = reinterpret_cast<floatx4*>(x + src * d);
  const bool adds = d1 || d2 || bias;
  floatx4 v[KEEP];
#pragma unroll
  for (int it = 0; it < KEEP; ++it) {
    const int c = tid + it * kGroupNormThreads;
    v[it] = c < chunks ? xr[c] : floatx4{0.f, 0.f, 0.f, 0.f};
  }
  if (adds) {
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c = tid + it * kGroupNormThreads;
      if (c >= chunks) continue;
      floatx4 s = {0.f, 0.f, 0.f, 0.f};
      if (d1)
        for (int k = 0; k < ns1; ++k) s += *reinterpret_cast<const floatx4*>(d1 + src * d + 4 * c + k * st1);
      if (d2)
        for (int k = 0; k < ns2; ++k) s += *reinterpret_cast<const floatx4*>(d2 + src * d + 4 * c + k * st2);
      if (bias) s += *reinterpret_cast<const floatx4*>(bias + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[it][e] = fmaf(mult, s[e], v[it][e]);
      if (write_x) xr[c] = v[it];
    }
  }
  if (!out) return;
  const int gsz = d / groups;
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < KEEP; ++it) {
      const int c = tid + it * kGroupNormThreads;
      if (c < chunks && (4 * c) / gsz == g)
#pragma unroll
        for (int e = 0; e < 4; ++e) ss = fmaf(v[it][e], v[it][e], ss);
    }
    ss = block_sum(ss, red);
    if (tid == 0) rstd_g[g] = 1.f / sqrtf(ss / (float)gsz + eps);
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < KEEP; ++it) {
    const int c = tid + it * kGroupNormThreads;
    if (c >= chunks) continue;
    const float rstd = rstd_g[(4 * c) / gsz];
    const floatx4 wv = *reinterpret_cast<const floatx4*>(w + 4 * c);
    TOUT o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = from_f32<TOUT>(v[it][e] * rstd * wv[e]);
    TOUT* dst = out + r * d + 4 * c;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[e] = o[e];
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_add_sinusoid(float* x, const int* positions, int n, int d, double base, hipStream_t stream) {
  KLLM_REQUIRE(x && positions, "add_sinusoid: null pointer");
  KLLM_REQUIRE(n > 0 && d > 0 && base > 0.0, "add_sinusoid: bad sizes n=%d d=%d base=%g", n, d, base);
  const long count = (long)n * ((d + 1) / 2);
  hipLaunchKernelGGL(add_sinusoid_kernel, dim3(ceil_div(count, 256)), dim3(256), 0, stream, x, positions, n, d,
                     log(base));
  KLLM_CHECK_LAUNCH("add_sinusoid");
  return 0;
}

extern "C" int kllm_unary_act(const float* in, int nsplit, long split_stride, int in_row_stride, void* out,
                              int out_dtype, int n, int f, int act, const float* params, hipStream_t stream) {
  KLLM_REQUIRE(in_row_stride >= f, "unary_act: rows of %d elements every %d", f, in_row_stride);
  KLLM_REQUIRE(in && out, "unary_act: null pointer");
  KLLM_REQUIRE(n > 0 && f > 0 && nsplit >= 1, "unary_act: bad sizes n=%d f=%d nsplit=%d", n, f, nsplit);
  KLLM_REQUIRE(act >= 0 && act < UNARY_ACT_COUNT, "unary_act: unknown activation %d", act);
  KLLM_REQUIRE(act != ACT_XIELU || params, "unary_act: this activation needs its two constants");
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "unary_act: unknown dtype %d", out_dtype);
  const long count = (long)n * f;
  const dim3 grid(ceil_div(count, 256));
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(unary_act_kernel<float>, grid, dim3(256), 0, stream, in, nsplit, split_stride, in_row_stride, f,
                       (float*)out, count, act, params);
  else
    hipLaunchKernelGGL(unary_act_kernel<bf16_t>, grid, dim3(256), 0, stream, in, nsplit, split_stride, in_row_stride, f,
                       (bf16_t*)out, count, act, params);
  KLLM_CHECK_LAUNCH("unary_act");
  return 0;
}

extern "C" int kllm_group_norm_add(float* x, const float* d1, int ns1, long st1, const float* d2, int ns2, long st2,
                                   const float* bias, float mult, const float* w, void* out, int out_dtype,
                                   const int* rows, int n, int d, int groups, float eps, int write_x,
                                   hipStream_t stream) {
  KLLM_REQUIRE(x, "group_norm_add: null pointer");
  KLLM_REQUIRE(n > 0 && d > 0 && groups > 0 && d % groups == 0, "group_norm_add: %d channels in %d groups (n=%d)", d,
               groups, n);
  KLLM_REQUIRE(!out || w, "group_norm_add: an output needs the norm's weight");
  KLLM_REQUIRE(!(rows && write_x), "group_norm_add: chosen rows are read only");
  KLLM_REQUIRE((!d1 || ns1 >= 1) && (!d2 || ns2 >= 1), "group_norm_add: a sum needs at least one slice");
  KLLM_REQUIRE(out_dtype == DT_F32 || out_dtype == DT_BF16, "group_norm_add: unknown dtype %d", out_dtype);
  const bool aligned = ((uintptr_t)x & 15) == 0 && (!d1 || (((uintptr_t)d1 & 15) == 0 && st1 % 4 == 0)) &&
                       (!d2 || (((uintptr_t)d2 & 15) == 0 && st2 % 4 == 0)) && (!bias || ((uintptr_t)bias & 15) == 0) &&
                       (!w || ((uintptr_t)w & 15) == 0);
  if (aligned && d % 4 == 0 && (d / groups) % 4 == 0 && groups <= kGroupNormMaxGroups && d <= 4 * kGroupNormThreads * 8) {
    const int keep = ceil_div(d / 4, kGroupNormThreads);
#define KLLM_GN(T, KEEP)                                                                                          \
  hipLaunchKernelGGL((group_norm_add_vec_kernel<T, KEEP>), dim3(n), dim3(kGroupNormThreads), 0, stream, x, d1, ns1, \
                     st1, d2, ns2, st2, bias, mult, w, (T*)out, rows, d, groups, eps, write_x)
    if (out_dtype == DT_F32) {
      if (keep <= 1) KLLM_GN(float, 1); else if (keep <= 2) KLLM_GN(float, 2); else if (keep <= 4) KLLM_GN(float, 4); else KLLM_GN(float, 8);
    } else {
      if (keep <= 1) KLLM_GN(bf16_t, 1); else if (keep <= 2) KLLM_GN(bf16_t, 2); else if (keep <= 4) KLLM_GN(bf16_t, 4); else KLLM_GN(bf16_t, 8);
    }
#undef KLLM_GN
    KLLM_CHECK_LAUNCH("group_norm_add");
    return 0;
  }
  int segs = 1;
  while (groups * segs < kGroupNormThreads / kWave && d / groups / (2 * segs) >= kWave) segs *= 2;
  const size_t lds = ((size_t)d + (size_t)groups * segs) * sizeof(float);
  KLLM_REQUIRE(lds <= 64 * 1024, "group_norm_add: a row of %d channels in %d groups does not fit into LDS", d, groups);
  if (out_dtype == DT_F32)
    hipLaunchKernelGGL(group_norm_add_kernel<float>, dim3(n), dim3(kGroupNormThreads), lds, stream, x, d1, ns1, st1,
                       d2, ns2, st2, bias, mult, w, (float*)out, rows, d, groups, segs, eps, write_x);
  else
    hipLaunchKernelGGL(group_norm_add_kernel<bf16_t>, dim3(n), dim3(kGroupNormThreads), lds, stream, x, d1, ns1, st1,
                       d2, ns2, st2, bias, mult, w, (bf16_t*)out, rows, d, groups, segs, eps, write_x);
  KLLM_CHECK_LAUNCH("group_norm_add");
  return 0;
}
