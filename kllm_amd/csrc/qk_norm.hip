// What lies between the query/key product and attention for a mixer whose values are its
// keys: biases, an RMS norm over the whole query projection and one over the whole key
// projection (all heads at once), a query temperature that grows with the position, and the
// append to the pages.  The key as projected (bias added, before its norm) is cached as the
// value, its normalised form as the key.  One workgroup per token, all in 32-bit.
//
// Page layout, per page and KV head: keys [slot][hd], values [hd][slot].
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kQkThreads = 256;

template <typename T>
__global__ __launch_bounds__(kQkThreads) void qk_norm_append_kernel(
    const float* __restrict__ qk, int nsplit, long split_stride, const float* __restrict__ q_bias,
    const float* __restrict__ k_bias, const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    float temp_coef, int temp_every, T* __restrict__ q_out, T* __restrict__ cache, const int* __restrict__ positions,
    const int* __restrict__ span_of_token, const int* __restrict__ block_table, int max_pages, int page_size, int H,
    int KV, int hd) {
  extern __shared__ float row[];            // [H*hd + KV*hd] the sums, then as many norm weights
  __shared__ float red[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int qd = H * hd, kd = KV * hd, cols = qd + kd;
  const float* in = qk + (long)t * cols;
  float* wrow = row + cols;
  float ssq = 0.f, ssk = 0.f;
  // eight of a thread's elements at a time: their loads (every slice, the bias) go out together
  for (int i0 = tid; i0 < cols; i0 += 8 * kQkThreads) {
    float v[8], wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kQkThreads;
      v[u] = 0.f;
      wv[u] = 1.f;
      if (i < cols) {
        if (i < qd) {
          if (q_w) wv[u] = q_w[i];
        } else if (k_w) {
          wv[u] = k_w[i - qd];
        }
        if (i < qd) {
          if (q_bias) v[u] = q_bias[i];
        } else if (k_bias) {
          v[u] = k_bias[i - qd];
        }
      }
    }
    for (int s = 0; s < nsplit; ++s)
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * kQkThreads;
        v[u] += i < cols ? in[i + s * split_stride] : 0.f;
      }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kQkThreads;
      if (i >= cols) continue;
      if (i < qd) ssq = fmaf(v[u], v[u], ssq); else ssk = fmaf(v[u], v[u], ssk);
      row[i] = v[u];
      wrow[i] = wv[u];
    }
  }
  ssq = block_sum(ssq, red);
  ssk = block_sum(ssk, red);
  const int pos = positions[t];
  float qmul = 1.f;
  if (temp_every > 0) qmul = 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f);
  const float rq = q_w ? 1.f / sqrtf(ssq / (float)qd + eps) : 1.f;
  const float rk = k_w ? 1.f / sqrtf(ssk / (float)kd + eps) : 1.f;
#pragma unroll 4
  for (int i = tid; i < qd; i += kQkThreads) {
    float v = row[i];
    if (q_w) v = v * rq * wrow[i];
    q_out[(long)t * qd + i] = from_f32<T>(v * qmul);
  }
  if (!cache) return;
  const int page = block_table[(long)span_of_token[t] * max_pages + pos / page_size];
  const int slot = pos % page_size;
  const long block = (long)page_size * hd;
  for (int i = tid; i < kd; i += kQkThreads) {
    const int kvh = i / hd, e = i % hd;
    const float raw = row[qd + i];
    const float key = k_w ? raw * rk * wrow[qd + i] : raw;
    T* kpage = cache + (((long)page * 2 + 0) * KV + kvh) * block;
    T* vpage = cache + (((long)page * 2 + 1) * KV + kvh) * block;
    kpage[(long)slot * hd + e] = from_f32<T>(key);
    vpage[(long)e * page_size + slot] = from_f32<T>(raw);
  }
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_qk_norm_append(const float* qk, int nsplit, long split_stride, const float* q_bias,
                                   const float* k_bias, const float* q_w, const float* k_w, float eps, float temp_coef,
                                   int temp_every, void* q_out, void* cache, const int* positions,
                                   const int* span_of_token, const int* block_table, int max_pages, int page_size,
                                   int n, int H, int KV, int hd, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(qk && q_out && positions, "qk_norm_append: null pointer");
  KLLM_REQUIRE(!cache || (span_of_token && block_table && max_pages > 0 && page_size > 0),
               "qk_norm_append: a cache needs its tables");
  KLLM_REQUIRE(n > 0 && H > 0 && KV > 0 && hd > 0 && nsplit >= 1, "qk_norm_append: bad sizes n=%d H=%d KV=%d hd=%d", n,
               H, KV, hd);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "qk_norm_append: unknown dtype %d", dtype);
  const size_t lds = 2 * (size_t)(H + KV) * hd * sizeof(float);
  KLLM_REQUIRE(lds <= 160 * 1024, "qk_norm_append: %d query and key channels do not fit into LDS", (H + KV) * hd);
  if (lds > 64 * 1024) {
    const void* fn = dtype == DT_F32 ? (const void*)qk_norm_append_kernel<float> : (const void*)qk_norm_append_kernel<bf16_t>;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) KLLM_FAIL((int)e, "qk_norm_append: cannot raise the LDS limit: %s", hipGetErrorString(e));
  }
  if (dtype == DT_F32)
    hipLaunchKernelGGL(qk_norm_append_kernel<float>, dim3(n), dim3(kQkThreads), lds, stream, qk, nsplit, split_stride,
                       q_bias, k_bias, q_w, k_w, eps, temp_coef, temp_every, (float*)q_out, (float*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd);
  else
    hipLaunchKernelGGL(qk_norm_append_kernel<bf16_t>, dim3(n), dim3(kQkThreads), lds, stream, qk, nsplit, split_stride,
                       q_bias, k_bias, q_w, k_w, eps, temp_coef, temp_every, (bf16_t*)q_out, (bf16_t*)cache, positions,
                       span_of_token, block_table, max_pages, page_size, H, KV, hd);
  KLLM_CHECK_LAUNCH("qk_norm_append");
  return 0;
}
