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
    const TW* __restrict__ w2, const float* __restrict__ w0, const float* __restrict__ low, int low_nsplit,
    long low_stride, float decay_scale, float key_eps, float* __restrict__ scan_in, float* __restrict__ gate, int H,
    int hd, int L) {
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
  if (!low)
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
    if (low) {                               // the low-rank path's second product was made by a matrix kernel
      for (int sl = 0; sl < low_nsplit; ++sl) lr += low[(long)t * HD + c + sl * low_stride];
    } else {
      const TW* w2r = w2 + (long)c * L;
      for (int l = 0; l < L; ++l) lr = fmaf(to_f32(w2r[l]), tl[l], lr);
    }
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

// The recurrence.  Columns of the state (value channels) do not see each other, so a workgroup
// takes a block of columns of one (span, head): thread (j, p) holds rows [8p, 8p + 8) of column
// j, the PARTS threads of a column are neighbouring lanes of one wave.  A token's vectors are
// the same for every column; they are staged through LDS, kScanBlock(hd) tokens at a time and
// the next block's loads in flight while this block's tokens are worked through, so that the
// chain from token to token holds arithmetic and LDS reads only.  Rows beyond hd are padding:
// their vectors are zero in LDS and their state stays zero.
constexpr int kScanThreads = 256;
constexpr int kScanRows = 8;
constexpr int kScanStage = 12;            // elements of a block that a thread stages, at most

__host__ __device__ inline int scan_block_tokens(int hd_pad) { return hd_pad >= 512 ? 1 : 512 / hd_pad; }

template <int PARTS>
__global__ __launch_bounds__(kScanThreads) void delta_scan_kernel(
    const float* __restrict__ scan_in, float* __restrict__ o_out, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ span_start, const int* __restrict__ span_pos, int H,
    int hd) {
  constexpr int NR = kScanRows;
  constexpr int HP = PARTS * NR;                       // rows with padding
  constexpr int COLS = kScanThreads / PARTS;           // columns of a workgroup
  constexpr int TB = HP >= 512 ? 1 : 512 / HP;         // tokens of a block
  constexpr int VEC = kScanFields * HP;                // floats of a token in LDS
  __shared__ __attribute__((aligned(16))) float tok[2 * TB * VEC];
  const int span = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int j = blockIdx.z * COLS + tid / PARTS, p = tid % PARTS;
  const bool col = j < hd;
  const int row0 = p * NR;
  float* S = state + ((long)slots[span] * H + h) * hd * hd;
  const int t0 = span_start[span], t1 = span_start[span + 1];
  const bool fresh = span_pos[span] == 0;
  float s[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int r = row0 + i;
    s[i] = (col && r < hd && !fresh) ? S[(long)r * hd + j] : 0.f;
  }
  if (HP != hd)
    for (int i = tid; i < 2 * TB * VEC; i += kScanThreads) tok[i] = 0.f;
  const int per_tok = kScanFields * hd;                // floats of a token in memory
  const long tok_stride = (long)H * per_tok;
  const float* base = scan_in + (long)h * per_tok;
  float pre[kScanStage];
  auto ask = [&](int first, int count) {               // the block's elements into registers
#pragma unroll
    for (int k = 0; k < kScanStage; ++k) {
      const int idx = tid + k * kScanThreads;
      const int tt = idx / per_tok, e = idx % per_tok;
      pre[k] = (tt < count) ? base[(long)(first + tt) * tok_stride + e] : 0.f;
    }
  };
  auto put = [&](float* buf, int count) {
#pragma unroll
    for (int k = 0; k < kScanStage; ++k) {
      const int idx = tid + k * kScanThreads;
      const int tt = idx / per_tok, e = idx % per_tok;
      if (tt < count) buf[tt * VEC + (e / hd) * HP + e % hd] = pre[k];
    }
  };
  __syncthreads();                                     // the padding is zero before anything is staged
  ask(t0, min(TB, t1 - t0));
  put(tok, min(TB, t1 - t0));
  __syncthreads();
  int which = 0;
  for (int tb = t0; tb < t1; tb += TB, which ^= 1) {
    const int count = min(TB, t1 - tb);
    const int next_count = min(TB, t1 - tb - TB);      // <= 0: this is the last block
    if (next_count > 0) ask(tb + TB, next_count);
    const float* buf = tok + which * TB * VEC;
    for (int tt = 0; tt < count; ++tt, buf += VEC) {
      const floatx4* r4 = reinterpret_cast<const floatx4*>(buf + row0);
      const floatx4* k4 = reinterpret_cast<const floatx4*>(buf + HP + row0);
      const floatx4* w4 = reinterpret_cast<const floatx4*>(buf + 3 * HP + row0);
      const floatx4* u4 = reinterpret_cast<const floatx4*>(buf + 4 * HP + row0);
      const floatx4* a4 = reinterpret_cast<const floatx4*>(buf + 5 * HP + row0);
      const float vj = buf[2 * HP + (col ? j : 0)];
      float us = 0.f;
#pragma unroll
      for (int c = 0; c < NR / 4; ++c) {
        const floatx4 u = u4[c];
#pragma unroll
        for (int e = 0; e < 4; ++e) us = fmaf(u[e], s[4 * c + e], us);
      }
#pragma unroll
      for (int off = 1; off < PARTS; off <<= 1) us += __shfl_xor(us, off, kWave);
      float o = 0.f;
#pragma unroll
      for (int c = 0; c < NR / 4; ++c) {
        const floatx4 w = w4[c], k = k4[c], a = a4[c], r = r4[c];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float sn = fmaf(w[e], s[4 * c + e], fmaf(k[e], vj, -a[e] * us));
          s[4 * c + e] = sn;
          o = fmaf(sn, r[e], o);
        }
      }
#pragma unroll
      for (int off = 1; off < PARTS; off <<= 1) o += __shfl_xor(o, off, kWave);
      if (col && p == 0) o_out[((long)(tb + tt) * H + h) * hd + j] = o;
    }
    if (next_count > 0) put(tok + (which ^ 1) * TB * VEC, next_count);
    __syncthreads();                                   // the next block is staged; this one is done with
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
                               const float* w0, const float* low, int low_nsplit, long low_stride, float decay_scale,
                               float key_eps, float* scan_in, float* gate, int n, int H, int hd, int L, int w_dtype,
                               hipStream_t stream) {
  KLLM_REQUIRE(proj && a_bias && (w2 || low) && w0 && scan_in && gate, "delta_prep: null pointer");
  KLLM_REQUIRE(!low || low_nsplit >= 1, "delta_prep: the low-rank sums need at least one slice");
  KLLM_REQUIRE(n > 0 && H > 0 && hd > 0 && L > 0 && nsplit >= 1, "delta_prep: bad sizes n=%d H=%d hd=%d L=%d", n, H, hd,
               L);
  KLLM_REQUIRE(w_dtype == DT_F32 || w_dtype == DT_BF16, "delta_prep: unknown dtype %d", w_dtype);
  const size_t lds = ((size_t)L + (size_t)H * hd + H) * sizeof(float);
  KLLM_REQUIRE(lds <= 64 * 1024, "delta_prep: %d channels do not fit into LDS", H * hd);
  if (w_dtype == DT_F32)
    hipLaunchKernelGGL(delta_prep_kernel<float>, dim3(n), dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const float*)w2, w0, low, low_nsplit, low_stride, decay_scale, key_eps, scan_in, gate, H, hd, L);
  else
    hipLaunchKernelGGL(delta_prep_kernel<bf16_t>, dim3(n), dim3(kPrepThreads), lds, stream, proj, nsplit, split_stride,
                       a_bias, (const bf16_t*)w2, w0, low, low_nsplit, low_stride, decay_scale, key_eps, scan_in, gate, H, hd, L);
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
  // rows in eights over the lanes of a column: 8, 16, 32 ... 256 rows with padding
  int parts = 1;
  while (parts * kScanRows < hd) parts *= 2;
  const int cols = kScanThreads / parts;
  const dim3 grid(n_spans, H, ceil_div(hd, cols));
#define KLLM_SCAN(PARTS)                                                                                      \
  case PARTS:                                                                                                 \
    static_assert(kScanStage * kScanThreads >= (PARTS * kScanRows >= 512 ? 1 : 512 / (PARTS * kScanRows)) *   \
                                                   kScanFields * PARTS * kScanRows, "a block is staged whole"); \
    hipLaunchKernelGGL((delta_scan_kernel<PARTS>), grid, dim3(kScanThreads), 0, stream, scan_in, o_out, state, \
                       slots, span_start, span_pos, H, hd);                                                   \
    break
  switch (parts) {
    KLLM_SCAN(1); KLLM_SCAN(2); KLLM_SCAN(4); KLLM_SCAN(8); KLLM_SCAN(16); KLLM_SCAN(32);
    default: KLLM_FAIL(ERR_ARG, "delta_scan: heads of %d are not built", hd);
  }
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
