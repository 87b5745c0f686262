// Activations between the two matrix products of a feed-forward without a gate, in place or into another tensor:
//   1  gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
//   2  gelu(z) = 0.5 z (1 + erf(z / sqrt 2))
//   3  relu(z)^2
// in fp32, rounded once when stored.
#include "common.h"

enum { IA_ACT_GELU_TANH = 1, IA_ACT_GELU_ERF = 2, IA_ACT_RELU_SQUARED = 3 };

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(const T* __restrict__ in, T* __restrict__ out, size_t n,
                                                         int kind) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const float z = to_float(in[i]);
    float y = z;
    if (kind == IA_ACT_GELU_TANH) y = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));   // gelu_tanh_f below, same roundings
    else if (kind == IA_ACT_GELU_ERF) y = 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
    else if (kind == IA_ACT_RELU_SQUARED) { const float r = fmaxf(z, 0.f); y = r * r; }
    out[i] = from_float<T>(y);
  }
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// Eight bfloat16 values (16 bytes) a thread and pass.
__global__ __launch_bounds__(256) void gelu_tanh_bf16x8_kernel(const uint4* __restrict__ in, uint4* __restrict__ out,
                                                               size_t n8) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride) {
    const uint4 v = in[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = gelu_tanh_f(__uint_as_float(w[k] << 16)), hi = gelu_tanh_f(__uint_as_float(w[k] & 0xffff0000u));
      o[k] = (uint32_t)float_to_bf16_bits(lo) | ((uint32_t)float_to_bf16_bits(hi) << 16);
    }
    out[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

extern "C" int ia_activation(const void* in, void* out, int dtype, size_t n, int kind, hipStream_t stream) {
  if (kind < IA_ACT_GELU_TANH || kind > IA_ACT_RELU_SQUARED || (dtype != IA_F32 && dtype != IA_BF16)) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!in || !out) return IA_ERR_BAD_ARG;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (kind == IA_ACT_GELU_TANH && dtype == IA_BF16 && (n & 7) == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
    const size_t n8 = n >> 3;
    gelu_tanh_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256 < 65536 ? (n8 + 255) / 256 : 65536), 256, 0, stream>>>(
        (const uint4*)in, (uint4*)out, n8);
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
  if (dtype == IA_F32)
    activation_kernel<float><<<grid, 256, 0, stream>>>((const float*)in, (float*)out, n, kind);
  else
    activation_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, n, kind);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// x <- x * s over n fp32 values (logits that a model multiplies by a constant).
__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ x, size_t n, float s) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) x[i] *= s;
}

extern "C" int ia_scale(float* x, int rows, int cols, float s, hipStream_t stream) {
  if (rows < 0 || cols < 0) return IA_ERR_BAD_ARG;
  const size_t n = (size_t)rows * cols;
  if (n == 0) return IA_OK;
  if (!x) return IA_ERR_BAD_ARG;
  scale_kernel<<<(unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536), 256, 0, stream>>>(x, n, s);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_activation)
IA_OP(ia_scale)
