// RMSNorm on a branch's output, then the residual add: the arrangement in which a sublayer reads the residual
// stream itself and its result is normalised before it is added,
//   d = sum_k delta[k][n]  (fp32),   h[n] += d / sqrt(mean(d^2) + eps) * w,   x[n] = h[n] in the activations' type.
// delta is [splits, delta_rows, H]: one tensor in the activations' type, or a stack of fp32 partial sums (of a
// split matrix product, or of the experts a token was routed to), added in the order of their index.  x (nullable)
// is what the next sublayer's matrix products read.  All arithmetic is fp32; the row's sums are taken in one
// order whatever the batch holds.
#include "common.h"

#define NB_NT 256
#define NB_KEEP 16      // values of a row that a thread keeps in registers: rows up to NB_NT * NB_KEEP are read once

template <typename TD, typename TX>
__global__ __launch_bounds__(NB_NT) void norm_add_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                         int splits, size_t split_stride,
                                                         const void* __restrict__ w, int w_dtype,
                                                         TX* __restrict__ x, int H, float eps) {
  __shared__ float red[NB_NT / 64];
  const int row = blockIdx.x;
  const TD* dr = delta + (size_t)row * H;
  float* hr = h + (size_t)row * H;
  float keep[NB_KEEP];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NB_KEEP; ++c) {
    const int i = threadIdx.x + c * NB_NT;
    keep[c] = 0.f;
    if (i < H) {
      keep[c] = load_split_sum(dr + i, splits, split_stride);
      ss = fmaf(keep[c], keep[c], ss);
    }
  }
  for (int i = threadIdx.x + NB_KEEP * NB_NT; i < H; i += NB_NT) {      // wider rows: the rest is read twice
    const float d = load_split_sum(dr + i, splits, split_stride);
    ss = fmaf(d, d, ss);
  }
  ss = block_sum<NB_NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
  for (int c = 0; c < NB_KEEP; ++c) {
    const int i = threadIdx.x + c * NB_NT;
    if (i < H) {
      const float s = hr[i] + keep[c] * inv * load_as_float(w, w_dtype, i);
      hr[i] = s;
      if (x) x[(size_t)row * H + i] = from_float<TX>(s);
    }
  }
  for (int i = threadIdx.x + NB_KEEP * NB_NT; i < H; i += NB_NT) {
    const float d = load_split_sum(dr + i, splits, split_stride);
    const float s = hr[i] + d * inv * load_as_float(w, w_dtype, i);
    hr[i] = s;
    if (x) x[(size_t)row * H + i] = from_float<TX>(s);
  }
}

// delta_dtype: type of delta (IA_F32 for partial sums); act_dtype: type of x.  delta is [splits, delta_rows, H].
extern "C" int ia_norm_add(float* h, const void* delta, int delta_dtype, int splits, int delta_rows, const void* w,
                           int w_dtype, void* x, int act_dtype, int N, int H, float eps, hipStream_t stream) {
  if (N < 0 || H <= 0 || !(eps > 0.f) || !delta || !h || !w || splits < 1 || delta_rows < N) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  const size_t stride = (size_t)delta_rows * H;
  if (delta_dtype == IA_F32 && act_dtype == IA_F32)
    norm_add_kernel<float, float><<<N, NB_NT, 0, stream>>>(h, (const float*)delta, splits, stride, w, w_dtype,
                                                           (float*)x, H, eps);
  else if (delta_dtype == IA_BF16 && act_dtype == IA_BF16)
    norm_add_kernel<bf16_t, bf16_t><<<N, NB_NT, 0, stream>>>(h, (const bf16_t*)delta, splits, stride, w, w_dtype,
                                                             (bf16_t*)x, H, eps);
  else if (delta_dtype == IA_F32 && act_dtype == IA_BF16)
    norm_add_kernel<float, bf16_t><<<N, NB_NT, 0, stream>>>(h, (const float*)delta, splits, stride, w, w_dtype,
                                                            (bf16_t*)x, H, eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_norm_add)
