// Activations between the two matrix products of a feed-forward without a gate, in place or into another tensor:
//   gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
// in fp32, rounded once when stored.
#include "common.h"

enum { IA_ACT_GELU_TANH = 1 };

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(const T* __restrict__ in, T* __restrict__ out, size_t n,
                                                         int kind) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const float z = to_float(in[i]);
    float y = z;
    if (kind == IA_ACT_GELU_TANH) y = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    out[i] = from_float<T>(y);
  }
}

extern "C" int ia_activation(const void* in, void* out, int dtype, size_t n, int kind, hipStream_t stream) {
  if (kind != IA_ACT_GELU_TANH || (dtype != IA_F32 && dtype != IA_BF16)) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!in || !out) return IA_ERR_BAD_ARG;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (dtype == IA_F32)
    activation_kernel<float><<<grid, 256, 0, stream>>>((const float*)in, (float*)out, n, kind);
  else
    activation_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, n, kind);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_activation)
