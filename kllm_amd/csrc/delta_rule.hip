// A recurrent mixer with a matrix state per head, updated by a generalized delta rule:
//
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        o_t = S_t^T r_t
//
// with u_t the key divided by its length, w_t a decay per key channel and a_t a removal rate
// per key channel.  S is [key channel][value channel], 32-bit, one per request and head, kept
// in a state slot between steps and started from zero at position 0.
//
// Three kernels: `prep` turns the projections' sums into what the recurrence reads (per token,
// parallel), `scan` runs the recurrence (per request and head, token after token), `out`
// normalises each head's output, scales and gates it (per token, parallel).  Everything that
// enters the recurrence is 32-bit.
#include <math.h>

#include "common.hpp"
#include "kllm_kernels.h"

namespace kllm {

constexpr int kPrepThreads = 256;
// per (token, head): r, k, v, w, u, a*u, each hd floats
constexpr int kScanFields = 6;

// proj: [nsplit][n][5*HD + L], columns r | k | v | g | a | w1.
// scan_in: [n][H][6][hd]; gate: [n][HD] = sigmoid(g).
template <typename TW>
__global__ __launch_bounds__(kPrepThreads) void delta_prep_kernel(
    const float* __restrict__ proj, int nsplit, long split_stride, const float* __restrict__ a_bias,
    const TW* __restrict__ w2, const float* __restrict__ w0, float decay_scale, float key_eps,
    float* __restrict__ scan_in, float* __restrict__ gate, int H, int hd, int L) {
  extern __shared__ float lds[];           // [L] tanh of the low-rank input, [HD] keys, [H] sums of squares
  float* tl = lds;
  float* ks = lds + L;
  float* kss = ks + H * hd;
  const int t = blockIdx.x, tid = threadIdx.x;
  const int HD = H * hd, cols = 5 * HD + L;
  const float* in = proj + (long)t * cols;
  auto column = [&](int c) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += in[c + s * split_stride];
    return v;
  };
  for (int l = tid; l < L; l += kPrepThreads) tl[l] = tanhf(column(5 * HD + l));
  for (int c = tid; c < HD; c += kPrepThreads) ks[c] = column(HD + c);
  __syncthreads();
  const int lane = tid % kWave, wave = tid / kWave;
  for (int h = wave; h < H; h += kPrepThreads / kWave) {
    float ss = 0.f;
    for (int e = lane; e < hd; e += kWave) ss = fmaf(ks[h * hd + e], ks[h * hd + e], ss);
    ss = wave_sum(ss);
    if (lane == 0) kss[h] = ss;
  }
  __syncthreads();
  for (int c = tid; c < HD; c += kPrepThreads) {
    const int h = c / hd, e = c % hd;
    float lr = w0[c];
    const TW* w2r = w2 + (long)c * L;
    for (int l = 0; l < L; ++l) lr = fmaf(to_f32(w2r[l]), tl[l], lr);
    const float w = expf(-decay_scale * sigmoid_f32(lr));
    const float a = sigmoid_f32(column(4 * HD + c) + a_bias[c]);
    const float k = ks[c];
    const float u = k / sqrtf(kss[h] + key_eps);
    float* o = scan_in + (((long)t * H + h) * kScanFields) * hd + e;
    o[0 * hd] = column(c);
    o[1 * hd] = k;
    o[2 * hd] = column(2 * HD + c);
    o[3 * hd] = w;
    o[4 * hd] = u;
    o[5 * hd] = a * u;
    gate[(long)t * HD + c] = sigmoid_f32(column(3 * HD + c));
  }
}

// One workgroup per (span, head).  Thread (j, p) holds rows [p*RPT, (p+1)*RPT) of column j of
// the state; the PARTS threads of a column are neighbouring lanes.  NR = rows held by a thread.
template <int NR, int PARTS>
__global__ void delta_scan_kernel(const float* __restrict__ scan_in, float* __restrict__ o_out,
                                  float* __restrict__ state, const int* __restrict__ slots,
                                  const int* __restrict__ span_start, const int* __restrict__ span_pos, int H, int hd) {
  extern __shared__ float tok[];           // [2][6*hd] the token's vectors, two buffers in turn
  const int span = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int j = tid / PARTS, p = tid % PARTS;
  const bool col = j < hd;
  const int row0 = p * NR;
  float* S = state + ((long)slots[span] * H + h) * hd * hd;
  const int t0 = span_start[span], t1 = span_start[span + 1];
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = row0 + i;
    s[i] = (col && r < hd && span_pos[span] != 0) ? S[(long)r * hd + j] : 0.f;
  }
  const int nvec = kScanFields * hd;              // at most two elements a thread (the workgroup has 4 hd threads)
  const int e0 = tid, e1 = tid + blockDim.x;
  {
    const float* src = scan_in + ((long)t0 * H + h) * nvec;
    if (e0 < nvec) tok[e0] = src[e0];
    if (e1 < nvec) tok[e1] = src[e1];
  }
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    float* buf = tok + ((t - t0) & 1) * nvec;
    float* nxt = tok + ((t + 1 - t0) & 1) * nvec;
    // the next token's vectors are asked for now and put into LDS behind this token's arithmetic
    const bool more = t + 1 < t1;
    const float* src = scan_in + ((long)(more ? t + 1 : t) * H + h) * nvec;
    const float n0 = e0 < nvec ? src[e0] : 0.f;
    const float n1 = e1 < nvec ? src[e1] : 0.f;
    const float* r_ = buf;
    const float* k_ = buf + hd;
    const float* v_ = buf + 2 * hd;
    const float* w_ = buf + 3 * hd;
    const float* u_ = buf + 4 * hd;
    const float* au_ = buf + 5 * hd;
    float us = 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int r = row0 + i;
      if (r < hd) us = fmaf(u_[r], s[i], us);
    }
#pragma unroll
    for (int off = 1; off < PARTS; off <<= 1) us += __shfl_xor(us, off, kWave);
    const float vj = col ? v_[j] : 0.f;
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int r = row0 + i;
      if (r < hd) {
        s[i] = fmaf(w_[r], s[i], fmaf(k_[r], vj, -au_[r] * us));
        o = fmaf(s[i], r_[r], o);
      }
    }
#pragma unroll
    for (int off = 1; off < PARTS; off <<= 1) o += __shfl_xor(o, off, kWave);
    if (col && p == 0) o_out[((long)t * H + h) * hd + j] = o;
    if (more) {
      if (e0 < nvec) nxt[e0] = n0;
      if (e1 < nvec) nxt[e1] = n1;
    }
    __syncthreads();                        // the next token's vectors are staged; this one's are done with
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = row0 + i;
    if (col && r < hd) S[(long)r * hd + j] = s[i];
  }
}

// out[t][h*hd + e] = o / sqrt(mean over the head of o^2 + eps) * weight * gate, one wave per (token, head).
template <typename T>
__global__ void delta_out_kernel(const float* __restrict__ o, const float* __restrict__ gate,
                                 const float* __restrict__ weight, float eps, T* __restrict__ out, long heads_total,
                                 int H, int hd) {
  const long item = (long)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= heads_total) return;
  const int lane = threadIdx.x % kWave;
  const int h = (int)(item % H);
  const float* orow = o + item * hd;
  float ss = 0.f;
  for (int e = lane; e < hd; e += kWave) ss = fmaf(orow[e], orow[e], ss);
  ss = wave_sum(ss);
  const float rstd = 1.f / sqrtf(ss / (float)hd + eps);
  for (int e = lane; e < hd; e += kWave)
    out[item * hd + e] = from_f32<T>(orow[e] * rstd * weight[h * hd + e] * gate[item * hd + e]);
}

}  // namespace kllm

using namespace kllm;

extern "C" int kllm_delta_prep(const float* proj, int nsplit, long split_stride, const float* a_bias, const void* w2,
                               const float* w0, float decay_scale, float key_eps, float* scan_in, float* gate, int n,
                               int H, int hd, int L, int w_dtype, hipStream_t stream) {
  KLLM_REQUIRE(proj && a_bias && w2 && w0 && scan_in && gate, "delta_prep: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0 && L > 0 && nsplit >= 1, "delta_prep: bad sizes n=%d H=%d hd=%d L=%d", n, H, hd,
               L);
  KLLM_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "delta_prep: unknown dtype %d", w_dtype);
  const size_t lds = ((size_t)L + (size_t)H * hd + H) * sizeof(float);
  KLLM_REQUIRE(lds <= 64 * 1024, "delta_prep: %d channels do not fit into LDS", H * hd);
  if (w_dtype == DT_F32)
    hipLaunchKernelGGL(delta_prep_kernel<float>, dim3(n), dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const float*)w2, w0, decay_scale, key_eps, scan_in, gate, H, hd, L);
  else
    hipLaunchKernelGGL(delta_prep_kernel<bf16_t>, dim3(n), dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const bf16_t*)w2, w0, decay_scale, key_eps, scan_in, gate, H, hd, L);
  KLLM_CHECK_LAUNCH("delta_prep");
  return 0;
}

extern "C" int kllm_delta_scan_max_dim(void) { return 256; }

extern "C" int kllm_delta_scan(const float* scan_in, float* o_out, float* state, const int* slots,
                               const int* span_start, const int* span_pos, int n_spans, int H, int hd,
                               hipStream_t stream) {
  KLLM_REQUIRE(scan_in && o_out && state && slots && span_start && span_pos, "delta_scan: null pointer");
  KLLM_REQUIRE(n_spans > 0 && H > 0 && H <= 65535 && hd > 0 && hd <= 256, "delta_scan: bad sizes spans=%d H=%d hd=%d",
               n_spans, H, hd);
  const dim3 grid(n_spans, H);
  const size_t lds = 2 * (size_t)kScanFields * hd * sizeof(float);
  // every column's rows over four neighbouring lanes; a thread holds hd/4 rows, rounded up
#define KLLM_SCAN(NR)                                                                                             \
  hipLaunchKernelGGL((delta_scan_kernel<NR, 4>), grid, dim3(ceil_div(hd * 4, kWave) * kWave), lds, stream, scan_in, \
                     o_out, state, slots, span_start, span_pos, H, hd)
  if (hd <= 32) KLLM_SCAN(8);
  else if (hd <= 64) KLLM_SCAN(16);
  else if (hd <= 128) KLLM_SCAN(32);
  else KLLM_SCAN(64);
#undef KLLM_SCAN
  KLLM_CHECK_LAUNCH("delta_scan");
  return 0;
}

extern "C" int kllm_delta_out(const float* o, const float* gate, const float* weight, float eps, void* out, int n, int H,
                              int hd, int dtype, hipStream_t stream) {
  KLLM_REQUIRE(o && gate && weight && out, "delta_out: null pointer");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0, "delta_out: bad sizes n=%d H=%d hd=%d", n, H, hd);
  KLLM_REQUIRE(dtype == DT_F32 || dtype == DT_BF16, "delta_out: unknown dtype %d", dtype);
  const long total = (long)n * H;
  const dim3 grid(ceil_div(total, 4));
  if (dtype == DT_F32)
    hipLaunchKernelGGL(delta_out_kernel<float>, grid, dim3(256), 0, stream, o, gate, weight, eps, (float*)out, total, H,
                       hd);
  else
    hipLaunchKernelGGL(delta_out_kernel<bf16_t>, grid, dim3(256), 0, stream, o, gate, weight, eps, (bf16_t*)out, total,
                       H, hd);
  KLLM_CHECK_LAUNCH("delta_out");
  return 0;
}
