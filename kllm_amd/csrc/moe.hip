// A routed feed-forward (mixture of experts) whose launches depend on the step's shape only:
// which token goes to which expert stays on the device.
//
//   kllm_moe_route    per token: softmax of the router's sums over all experts, the `top` largest
//                     of (score + correction), their scores divided by their sum
//   kllm_moe_plan     the (token, choice) entries grouped by expert, and a list of tiles of up to
//                     32 entries of one expert (a fixed number of tiles, the unused ones empty)
//   kllm_moe_expert   one tile's product with its expert's weights on the matrix cores (32 x 32
//                     per wave, 32-bit or bfloat16 operands straight from memory): gate and up
//                     with the gate in the epilogue, or down
//   kllm_moe_combine  per token the weighted sum of its choices' outputs, in the order of the
//                     choices; an expert beyond the last real one is the identity (its output is
//                     the feed-forward's input); plus the sums of a shared expert
//
// A row's result depends on the row alone: on no other entry of its tile and not on where in
// the tile it lies.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kMoeTileRows = 32;

__global__ void moe_route_kernel(const float* __restrict__ z, int nsplit, long split_stride,
                                 const float* __restrict__ correction, int n, int R, int top, int* __restrict__ idx,
                                 float* __restrict__ wgt) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  auto z_at = [&](int e) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += z[s * split_stride + (long)t * R + e];
    return v;
  };
  float m = -INFINITY;
  for (int e = 0; e < R; ++e) m = fmaxf(m, z_at(e));
  float den = 0.f;
  for (int e = 0; e < R; ++e) den += expf(z_at(e) - m);
  float picked = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = 0;
    float best_choice = -INFINITY, best_score = 0.f;
    for (int e = 0; e < R; ++e) {
      bool taken = false;
      for (int j = 0; j < k; ++j) taken |= idx[(long)t * top + j] == e;
      if (taken) continue;
      const float s = expf(z_at(e) - m) / den;
      const float c = correction ? s + correction[e] : s;
      if (c > best_choice) {
        best_choice = c;
        best_score = s;
        best = e;
      }
    }
    idx[(long)t * top + k] = best;
    wgt[(long)t * top + k] = best_score;
    picked += best_score;
  }
  const float inv = 1.f / (picked + 1e-20f);
  for (int k = 0; k < top; ++k) wgt[(long)t * top + k] *= inv;
}

// One workgroup.  tiles: [max_tiles][3] = (expert, first place in `sorted`, entries).
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ idx, int entries, int E, int max_tiles,
                                                        int* __restrict__ sorted, int* __restrict__ tiles) {
  extern __shared__ int plan_lds[];
  int* counts = plan_lds;
  int* offs = plan_lds + E;
  int* cursor = plan_lds + 2 * E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = cursor[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < entries; i += blockDim.x) {
    const int e = idx[i];
    if (e < E) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      offs[e] = off;
      for (int s = 0; s < counts[e] && nt < max_tiles; s += kMoeTileRows, ++nt) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = off + s;
        tiles[3 * nt + 2] = min(kMoeTileRows, counts[e] - s);
      }
      off += counts[e];
    }
    for (; nt < max_tiles; ++nt) tiles[3 * nt] = tiles[3 * nt + 1] = tiles[3 * nt + 2] = 0;
  }
  __syncthreads();
  // Which place an entry gets among its expert's is left to the order of arrival: a row's
  // result does not depend on it.
  for (int i = threadIdx.x; i < entries; i += blockDim.x) {
    const int e = idx[i];
    if (e < E) sorted[offs[e] + atomicAdd(&cursor[e], 1)] = i;
  }
}

template <typename T> struct MoeOperand;
template <> struct MoeOperand<bf16_t> { typedef bf16x8 type; };
template <> struct MoeOperand<float> { typedef floatx4 type; };

__device__ __forceinline__ floatx16 moe_mfma(bf16x8 a, bf16x8 b, floatx16 acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ floatx16 moe_mfma(floatx4 a, floatx4 b, floatx16 acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc, 0, 0, 0);
  return acc;
}

// Sixteen bytes of a row from element k0 on; zeros beyond the row's end.  `vec`: rows are
// multiples of 16 bytes long, so a chunk is whole or absent and 16-byte loads are aligned.
template <typename T>
__device__ __forceinline__ typename MoeOperand<T>::type moe_chunk(const T* __restrict__ row, int k0, int K, bool vec) {
  typedef typename MoeOperand<T>::type op_t;
  constexpr int EPC = 16 / sizeof(T);
  op_t v;
  if (vec) {
    if (k0 < K) return *reinterpret_cast<const op_t*>(row + k0);
#pragma unroll
    for (int j = 0; j < EPC; ++j) v[j] = (T)0.f;
    return v;
  }
#pragma unroll
  for (int j = 0; j < EPC; ++j) v[j] = k0 + j < K ? row[k0 + j] : (T)0.f;
  return v;
}

// MODE 0: X is the feed-forward's input [tokens, K]; W [E][2 M][K], an expert's gate rows, then its
//         up rows; out [entries, M] in T: the gated activation.
// MODE 1: X is [entries, K]; W [E][M][K]; out [entries, M] float32.
// Grid (tiles, column blocks of 128); a wave takes 32 columns.  A lane's share of K: of every
// 128 bytes of a row, lanes 0-31 take the first 64 for their row and lanes 32-63 the other 64,
// four products of 16 bytes each; both operands are cut alike, which is all a product asks.
template <typename T, int MODE>
__global__ __launch_bounds__(256) void moe_expert_kernel(const T* __restrict__ X, const T* __restrict__ W,
                                                         void* __restrict__ out_, const int* __restrict__ sorted,
                                                         const int* __restrict__ tiles, int top, int M, int K, int act,
                                                         float limit, float alpha) {
  typedef typename MoeOperand<T>::type op_t;
  constexpr int EPC = 16 / sizeof(T);
  const int tile = blockIdx.x;
  const int count = tiles[3 * tile + 2];
  if (count == 0) return;
  const int expert = tiles[3 * tile], start = tiles[3 * tile + 1];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int c0 = (blockIdx.y * 4 + wave) * 32;
  if (c0 >= M) return;
  const int r = lane % 32, half = lane / 32;
  const int entry = sorted[start + (r < count ? r : 0)];
  const T* xrow = X + (long)(MODE == 0 ? entry / top : entry) * K;
  const int wr = min(c0 + r, M - 1);
  const T* wbase = W + (long)expert * (MODE == 0 ? 2 : 1) * M * K;
  const T* w0 = wbase + (long)wr * K;
  const T* w1 = wbase + (long)(M + wr) * K;      // MODE 0: the up row
  const bool vec = K % EPC == 0;
  floatx16 acc0, acc1;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc0[e] = acc1[e] = 0.f;
  constexpr int STEP = 8 * EPC;                  // elements of 128 bytes
  op_t a[4], b0[4], b1[4];
  auto load = [&](int k) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k0 = k + (half * 4 + i) * EPC;
      a[i] = moe_chunk<T>(xrow, k0, K, vec);
      b0[i] = moe_chunk<T>(w0, k0, K, vec);
      if (MODE == 0) b1[i] = moe_chunk<T>(w1, k0, K, vec);
    }
  };
  load(0);
  for (int k = 0; k < K; k += STEP) {
    op_t ca[4], cb0[4], cb1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ca[i] = a[i];
      cb0[i] = b0[i];
      if (MODE == 0) cb1[i] = b1[i];
    }
    if (k + STEP < K) load(k + STEP);            // the next 128 bytes are on their way during the products
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc0 = moe_mfma(ca[i], cb0[i], acc0);
      if (MODE == 0) acc1 = moe_mfma(ca[i], cb1[i], acc1);
    }
  }
  const int c = c0 + r;
  if (c >= M) return;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int row = 8 * (e / 4) + 4 * half + e % 4;
    if (row >= count) continue;
    const long dst = (long)sorted[start + row] * M + c;
    if (MODE == 0)
      reinterpret_cast<T*>(out_)[dst] = from_f32<T>(gated(acc0[e], acc1[e], act, limit, alpha));
    else
      reinterpret_cast<float*>(out_)[dst] = acc0[e];
  }
}

template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ y, const T* __restrict__ xin, const int* __restrict__ idx,
                                   const float* __restrict__ wgt, const float* __restrict__ shared, int ns,
                                   long shared_stride, float* __restrict__ out, long count, int d, int top, int E) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const long t = i / d;
  const int c = (int)(i % d);
  float v = 0.f;
  for (int s = 0; s < top; ++s) {
    const long entry = t * top + s;
    const float part = idx[entry] < E ? y[entry * d + c] : to_f32(xin[i]);
    v = fmaf(wgt[entry], part, v);
  }
  for (int s = 0; s < ns; ++s) v += shared[s * shared_stride + i];
  out[i] = v;
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_moe_tile_rows(void) { return kMoeTileRows; }

extern "C" int kllm_moe_route(const float* z, int nsplit, long split_stride, const float* correction, int n, int R,
                              int top, int* idx, float* wgt, hipStream_t stream) {
  KLLM_REQUIRE(z && idx && wgt, "moe_route: null pointer");
  KLLM_REQUIRE(n > 0 && R > 0 && top > 0 && top <= R && nsplit >= 1, "moe_route: bad sizes n=%d experts=%d top=%d", n, R,
               top);
  hipLaunchKernelGGL(moe_route_kernel, dim3(ceil_div(n, 64)), dim3(64), 0, stream, z, nsplit, split_stride, correction,
                     n, R, top, idx, wgt);
  KLLM_CHECK_LAUNCH("moe_route");
  return 0;
}

extern "C" int kllm_moe_plan(const int* idx, int entries, int E, int max_tiles, int* sorted, int* tiles,
                             hipStream_t stream) {
  KLLM_REQUIRE(idx && sorted && tiles, "moe_plan: null pointer");
  KLLM_REQUIRE(entries > 0 && E > 0 && E <= 4096, "moe_plan: bad sizes entries=%d experts=%d", entries, E);
  KLLM_REQUIRE(max_tiles >= ceil_div(entries, kMoeTileRows) + E, "moe_plan: %d tiles do not hold %d entries of %d experts",
               max_tiles, entries, E);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), stream, idx, entries, E,
                     max_tiles, sorted, tiles);
  KLLM_CHECK_LAUNCH("moe_plan");
  return 0;
}

extern "C" int kllm_moe_expert(const void* x, const void* w, void* out, const int* sorted, const int* tiles,
                               int max_tiles, int top, int m, int k, int mode, int act, float limit, float alpha,
                               int dtype, hipStream_t stream) {
  KLLM_REQUIRE(x && w && out && sorted && tiles, "moe_expert: null pointer");
  KLLM_REQUIRE(max_tiles > 0 && top > 0 && m > 0 && k > 0, "moe_expert: bad sizes tiles=%d top=%d m=%d k=%d", max_tiles,
               top, m, k);
  KLLM_REQUIRE(mode == 0 || mode == 1, "moe_expert: mode %d", mode);
  KLLM_REQUIRE(mode == 1 || gated_known(act), "moe_expert: unknown activation %d", act);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "moe_expert: unknown dtype %d", dtype);
  const dim3 grid(max_tiles, ceil_div(m, 128));
#define KLLM_MOE(T, MODE)                                                                                          \
  hipLaunchKernelGGL((moe_expert_kernel<T, MODE>), grid, dim3(256), 0, stream, (const T*)x, (const T*)w, out, sorted, \
                     tiles, top, m, k, act, limit, alpha)
  if (dtype == DT_F32) {
    if (mode == 0) KLLM_MOE(float, 0); else KLLM_MOE(float, 1);
  } else {
    if (mode == 0) KLLM_MOE(bf16_t, 0); else KLLM_MOE(bf16_t, 1);
  }
#undef KLLM_MOE
  KLLM_CHECK_LAUNCH("moe_expert");
  return 0;
}

extern "C" int kllm_moe_combine(const float* y, const void* xin, const int* idx, const float* wgt, const float* shared,
                                int ns, long shared_stride, float* out, int n, int d, int top, int E, int dtype,
                                hipStream_t stream) {
  KLLM_REQUIRE(y && xin && idx && wgt && out, "moe_combine: null pointer");
  KLLM_REQUIRE(n > 0 && d > 0 && top > 0 && E >= 0 && ns >= 0, "moe_combine: bad sizes n=%d d=%d top=%d", n, d, top);
  KLLM_REQUIRE(shared || ns == 0, "moe_combine: slices of a shared expert without its sums");
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "moe_combine: unknown dtype %d", dtype);
  const long count = (long)n * d;
  const dim3 grid(ceil_div(count, 256));
  if (dtype == DT_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, stream, y, (const float*)xin, idx, wgt, shared, ns,
                       shared_stride, out, count, d, top, E);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, dim3(256), 0, stream, y, (const bf16_t*)xin, idx, wgt, shared,
                       ns, shared_stride, out, count, d, top, E);
  KLLM_CHECK_LAUNCH("moe_combine");
  return 0;
}
