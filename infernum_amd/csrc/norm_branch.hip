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

// Rows of a multiple of 4 values up to NT * 4 * NV: every thread keeps its pieces of the row in registers, read 16
// (or 8) bytes at a time with the loads of all parts of a piece in flight together; one pass over memory.
__device__ __forceinline__ float4 nb_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 nb_load4(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void nb_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void nb_store4(bf16_t* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  u.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

template <typename TD, typename TX, int NT, int NV>
__global__ __launch_bounds__(NT) void norm_add_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                          int splits, size_t split_stride,
                                                          const void* __restrict__ w, int w_dtype,
                                                          TX* __restrict__ x, int H, float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const TD* dr = delta + (size_t)row * H;
  float* hr = h + (size_t)row * H;
  float4 d[NV], hv[NV], g[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    d[c] = hv[c] = g[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < H) {
      hv[c] = nb_load4(hr + i);
      g[c] = w_dtype == IA_F32 ? nb_load4((const float*)w + i) : nb_load4((const bf16_t*)w + i);
      d[c] = nb_load4(dr + i);
    }
  }
#pragma clang loop unroll_count(4)
  for (int k = 1; k < splits; ++k) {                 // the parts in the order of their index
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int i = (threadIdx.x + c * NT) * 4;
      if (i < H) {
        const float4 p = nb_load4(dr + k * split_stride + i);
        d[c].x += p.x; d[c].y += p.y; d[c].z += p.z; d[c].w += p.w;
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c)
    ss += __builtin_fmaf(d[c].x, d[c].x, d[c].y * d[c].y) + __builtin_fmaf(d[c].z, d[c].z, d[c].w * d[c].w);
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    if (i < H) {
      const float4 s = make_float4(hv[c].x + d[c].x * inv * g[c].x, hv[c].y + d[c].y * inv * g[c].y,
                                   hv[c].z + d[c].z * inv * g[c].z, hv[c].w + d[c].w * inv * g[c].w);
      nb_store4(hr + i, s);
      if (x) nb_store4(x + (size_t)row * H + i, s);
    }
  }
}

template <typename TD, typename TX>
static void launch_norm_add(float* h, const void* delta, int splits, size_t stride, const void* w, int w_dtype, void* x,
                            int N, int H, float eps, hipStream_t stream) {
  const TD* d = (const TD*)delta;
  TX* xo = (TX*)x;
  const bool aligned = ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(delta) |
                         reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15) == 0 &&
                       (stride & 3) == 0;
  if ((H & 3) == 0 && aligned && H <= 256 * 4)
    norm_add_vec_kernel<TD, TX, 256, 1><<<N, 256, 0, stream>>>(h, d, splits, stride, w, w_dtype, xo, H, eps);
  else if ((H & 3) == 0 && aligned && H <= 1024 * 4)      // the kernel follows from H alone: a row's sums are taken
    norm_add_vec_kernel<TD, TX, 1024, 1><<<N, 1024, 0, stream>>>(h, d, splits, stride, w, w_dtype, xo, H, eps);   // in one order
  else if ((H & 3) == 0 && aligned && H <= 1024 * 4 * 4)
    norm_add_vec_kernel<TD, TX, 1024, 4><<<N, 1024, 0, stream>>>(h, d, splits, stride, w, w_dtype, xo, H, eps);
  else
    norm_add_kernel<TD, TX><<<N, NB_NT, 0, stream>>>(h, d, splits, stride, w, w_dtype, xo, H, eps);
}

// delta_dtype: type of delta (IA_F32 for partial sums); act_dtype: type of x.  delta is [splits, delta_rows, H].
extern "C" int ia_norm_add(float* h, const void* delta, int delta_dtype, int splits, int delta_rows, const void* w,
                           int w_dtype, void* x, int act_dtype, int N, int H, float eps, hipStream_t stream) {
  if (N < 0 || H <= 0 || !(eps > 0.f) || !delta || !h || !w || splits < 1 || delta_rows < N) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  const size_t stride = (size_t)delta_rows * H;
  if (delta_dtype == IA_F32 && act_dtype == IA_F32)
    launch_norm_add<float, float>(h, delta, splits, stride, w, w_dtype, x, N, H, eps, stream);
  else if (delta_dtype == IA_BF16 && act_dtype == IA_BF16)
    launch_norm_add<bf16_t, bf16_t>(h, delta, splits, stride, w, w_dtype, x, N, H, eps, stream);
  else if (delta_dtype == IA_F32 && act_dtype == IA_BF16)
    launch_norm_add<float, bf16_t>(h, delta, splits, stride, w, w_dtype, x, N, H, eps, stream);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the same with a gate on the branch, and optionally the next sublayer's norm behind the add ----
//   d = sum_k delta[k][n] * sigmoid(gate[n] + gate_bias)   (fp32; the gate's logits in fp32 or the activations' type)
//   h[n] += d / sqrt(mean(d^2) + eps) * w
//   x[n] = h[n] / sqrt(mean(h[n]^2) + eps) * w_next   (with w_next; without it x[n] = h[n]; x may be absent)
// One workgroup a row, the row's values in registers (rows above NB_NT * NB_KEEP values are read again).
template <typename TD, typename TG, typename TX>
__global__ __launch_bounds__(NB_NT) void gated_norm_add_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                               int splits, size_t split_stride,
                                                               const TG* __restrict__ gate, int gate_stride,
                                                               int gate_splits, size_t gate_split_stride,
                                                               const float* __restrict__ gate_bias,
                                                               const void* __restrict__ w, int w_dtype,
                                                               const void* __restrict__ w_next, int w_next_dtype,
                                                               TX* __restrict__ x, int H, float eps) {
  __shared__ float red[NB_NT / 64];
  const int row = blockIdx.x;
  const TD* dr = delta + (size_t)row * H;
  const TG* gr = gate ? gate + (size_t)row * gate_stride : nullptr;
  float* hr = h + (size_t)row * H;
  auto gated = [&](int i) {
    float d = load_split_sum(dr + i, splits, split_stride);
    if (gr) {
      const float z = load_split_sum(gr + i, gate_splits, gate_split_stride) + (gate_bias ? gate_bias[i] : 0.f);
      d *= 1.0f / (1.0f + expf(-z));
    }
    return d;
  };
  float keep[NB_KEEP];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NB_KEEP; ++c) {
    const int i = threadIdx.x + c * NB_NT;
    keep[c] = 0.f;
    if (i < H) {
      keep[c] = gated(i);
      ss = fmaf(keep[c], keep[c], ss);
    }
  }
  for (int i = threadIdx.x + NB_KEEP * NB_NT; i < H; i += NB_NT) {
    const float d = gated(i);
    ss = fmaf(d, d, ss);
  }
  ss = block_sum<NB_NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  float s2 = 0.f;
#pragma unroll
  for (int c = 0; c < NB_KEEP; ++c) {
    const int i = threadIdx.x + c * NB_NT;
    if (i < H) {
      keep[c] = hr[i] + keep[c] * inv * load_as_float(w, w_dtype, i);
      hr[i] = keep[c];
      s2 = fmaf(keep[c], keep[c], s2);
    }
  }
  for (int i = threadIdx.x + NB_KEEP * NB_NT; i < H; i += NB_NT) {
    const float s = hr[i] + gated(i) * inv * load_as_float(w, w_dtype, i);
    hr[i] = s;
    s2 = fmaf(s, s, s2);
  }
  if (!x) return;
  float inv2 = 1.0f;
  if (w_next) {
    s2 = block_sum<NB_NT>(s2, red);
    inv2 = 1.0f / sqrtf(s2 / (float)H + eps);
  }
#pragma unroll
  for (int c = 0; c < NB_KEEP; ++c) {
    const int i = threadIdx.x + c * NB_NT;
    if (i < H) x[(size_t)row * H + i] = from_float<TX>(w_next ? keep[c] * inv2 * load_as_float(w_next, w_next_dtype, i) : keep[c]);
  }
  for (int i = threadIdx.x + NB_KEEP * NB_NT; i < H; i += NB_NT)
    x[(size_t)row * H + i] = from_float<TX>(w_next ? hr[i] * inv2 * load_as_float(w_next, w_next_dtype, i) : hr[i]);
}

// The same for rows of a multiple of 4 values up to NT * 4 * NV, with every pointer and stride a multiple of 16 bytes:
// a thread keeps its pieces of the row in registers, read 16 (or 8) bytes at a time, the loads of all parts of a piece
// in flight together; one pass over memory.  The sums of a row are taken in one order whatever the batch holds.
__device__ __forceinline__ float4 nb_load4_any(const void* p, int dtype, int i) {
  return dtype == IA_F32 ? nb_load4((const float*)p + i) : nb_load4((const bf16_t*)p + i);
}

template <typename TD, typename TG, typename TX, int NT, int NV>
__global__ __launch_bounds__(NT) void gated_norm_add_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                                int splits, size_t split_stride,
                                                                const TG* __restrict__ gate, int gate_stride,
                                                                int gate_splits, size_t gate_split_stride,
                                                                const float* __restrict__ gate_bias,
                                                                const void* __restrict__ w, int w_dtype,
                                                                const void* __restrict__ w_next, int w_next_dtype,
                                                                TX* __restrict__ x, int H, float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const TD* dr = delta + (size_t)row * H;
  float* hr = h + (size_t)row * H;
  float4 d[NV], hv[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    d[c] = hv[c] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < H) {
      hv[c] = nb_load4(hr + i);
      d[c] = nb_load4(dr + i);
    }
  }
#pragma clang loop unroll_count(4)
  for (int k = 1; k < splits; ++k) {                 // the parts in the order of their index
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int i = (threadIdx.x + c * NT) * 4;
      if (i < H) {
        const float4 p = nb_load4(dr + k * split_stride + i);
        d[c].x += p.x; d[c].y += p.y; d[c].z += p.z; d[c].w += p.w;
      }
    }
  }
  if (gate) {
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int i = (threadIdx.x + c * NT) * 4;
      if (i < H) {
        float4 z = nb_load4(gate + (size_t)row * gate_stride + i);
        for (int k = 1; k < gate_splits; ++k) {        // the logits' parts in the order of their index
          const float4 q = nb_load4(gate + k * gate_split_stride + (size_t)row * gate_stride + i);
          z.x += q.x; z.y += q.y; z.z += q.z; z.w += q.w;
        }
        if (gate_bias) {
          const float4 b = nb_load4(gate_bias + i);
          z.x += b.x; z.y += b.y; z.z += b.z; z.w += b.w;
        }
        d[c].x *= 1.0f / (1.0f + expf(-z.x));
        d[c].y *= 1.0f / (1.0f + expf(-z.y));
        d[c].z *= 1.0f / (1.0f + expf(-z.z));
        d[c].w *= 1.0f / (1.0f + expf(-z.w));
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c)
    ss += __builtin_fmaf(d[c].x, d[c].x, d[c].y * d[c].y) + __builtin_fmaf(d[c].z, d[c].z, d[c].w * d[c].w);
  ss = block_sum<NT>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  float s2 = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    if (i < H) {
      const float4 g = nb_load4_any(w, w_dtype, i);
      hv[c] = make_float4(hv[c].x + d[c].x * inv * g.x, hv[c].y + d[c].y * inv * g.y, hv[c].z + d[c].z * inv * g.z,
                          hv[c].w + d[c].w * inv * g.w);
      nb_store4(hr + i, hv[c]);
      s2 += __builtin_fmaf(hv[c].x, hv[c].x, hv[c].y * hv[c].y) + __builtin_fmaf(hv[c].z, hv[c].z, hv[c].w * hv[c].w);
    }
  }
  if (!x) return;
  float inv2 = 1.0f;
  if (w_next) {
    s2 = block_sum<NT>(s2, red);
    inv2 = 1.0f / sqrtf(s2 / (float)H + eps);
  }
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    if (i < H) {
      float4 o = hv[c];
      if (w_next) {
        const float4 g = nb_load4_any(w_next, w_next_dtype, i);
        o = make_float4(o.x * inv2 * g.x, o.y * inv2 * g.y, o.z * inv2 * g.z, o.w * inv2 * g.w);
      }
      nb_store4(x + (size_t)row * H + i, o);
    }
  }
}

template <typename TD, typename TG, typename TX>
static void launch_gated_norm_add_typed(float* h, const TD* delta, int splits, size_t stride, const TG* gate,
                                        int gate_stride, int gate_splits, size_t gate_split_stride, const float* gate_bias, const void* w, int w_dtype,
                                        const void* w_next, int w_next_dtype, TX* x, int N, int H, float eps,
                                        hipStream_t stream) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(delta) |
                         reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(gate_bias) |
                         reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(w_next) |
                         reinterpret_cast<uintptr_t>(x)) & 15) == 0 &&
                       (stride & 3) == 0 && (gate_stride & 3) == 0 && (gate_split_stride & 3) == 0 && (H & 3) == 0;
#define IA_GNA_VEC(NT, NV)                                                                                          \
  gated_norm_add_vec_kernel<TD, TG, TX, NT, NV><<<N, NT, 0, stream>>>(                                             \
      h, delta, splits, stride, gate, gate_stride, gate_splits, gate_split_stride, gate_bias, w, w_dtype, w_next,   \
      w_next_dtype, x, H, eps)
  if (aligned && H <= 256 * 4) IA_GNA_VEC(256, 1);           // the kernel follows from H alone: a row's sums are taken
  else if (aligned && H <= 1024 * 4) IA_GNA_VEC(1024, 1);    // in one order
  else if (aligned && H <= 1024 * 4 * 4) IA_GNA_VEC(1024, 4);
  else
    gated_norm_add_kernel<TD, TG, TX><<<N, NB_NT, 0, stream>>>(h, delta, splits, stride, gate, gate_stride, gate_splits,
                                                               gate_split_stride, gate_bias, w, w_dtype, w_next,
                                                               w_next_dtype, x, H, eps);
#undef IA_GNA_VEC
}

template <typename TD, typename TX>
static int launch_gated_norm_add(float* h, const void* delta, int splits, size_t stride, const void* gate, int gate_dtype,
                                 int gate_stride, int gate_splits, size_t gate_split_stride, const float* gate_bias, const void* w, int w_dtype, const void* w_next,
                                 int w_next_dtype, void* x, int N, int H, float eps, hipStream_t stream) {
  if (gate_dtype == IA_F32)
    launch_gated_norm_add_typed<TD, float, TX>(h, (const TD*)delta, splits, stride, (const float*)gate, gate_stride,
                                               gate_splits, gate_split_stride, gate_bias, w, w_dtype, w_next, w_next_dtype, (TX*)x, N, H, eps, stream);
  else if (gate_dtype == IA_BF16)
    launch_gated_norm_add_typed<TD, bf16_t, TX>(h, (const TD*)delta, splits, stride, (const bf16_t*)gate, gate_stride,
                                                gate_splits, gate_split_stride, gate_bias, w, w_dtype, w_next, w_next_dtype, (TX*)x, N, H, eps, stream);
  else
    return IA_ERR_BAD_ARG;
  return IA_OK;
}

// delta [splits, delta_rows, H] of delta_dtype; gate (nullable) [gate_splits, gate_rows, >= H] rows of gate_stride
// values of gate_dtype (parts of the logits, added in the order of their index; more than one part: fp32);
// gate_bias (nullable) fp32 [H]; w_next (nullable): the weight of the norm that follows the add; x (nullable) of act_dtype.
extern "C" int ia_gated_norm_add(float* h, const void* delta, int delta_dtype, int splits, int delta_rows, const void* gate,
                                 int gate_dtype, int gate_stride, int gate_splits, int gate_rows, const float* gate_bias, const void* w, int w_dtype,
                                 const void* w_next, int w_next_dtype, void* x, int act_dtype, int N, int H, float eps,
                                 hipStream_t stream) {
  if (N < 0 || H <= 0 || !(eps > 0.f) || !delta || !h || !w || splits < 1 || delta_rows < N ||
      (gate && (gate_stride < H || gate_splits < 1 || gate_rows < N || (gate_splits > 1 && gate_dtype != IA_F32))))
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  const size_t stride = (size_t)delta_rows * H;
  const size_t gstride = gate ? (size_t)gate_rows * gate_stride : 0;
  if (!gate) gate_splits = 1;
  int rc;
  if (delta_dtype == IA_F32 && act_dtype == IA_F32)
    rc = launch_gated_norm_add<float, float>(h, delta, splits, stride, gate, gate_dtype, gate_stride, gate_splits, gstride, gate_bias, w, w_dtype,
                                             w_next, w_next_dtype, x, N, H, eps, stream);
  else if (delta_dtype == IA_BF16 && act_dtype == IA_BF16)
    rc = launch_gated_norm_add<bf16_t, bf16_t>(h, delta, splits, stride, gate, gate_dtype, gate_stride, gate_splits, gstride, gate_bias, w,
                                               w_dtype, w_next, w_next_dtype, x, N, H, eps, stream);
  else if (delta_dtype == IA_F32 && act_dtype == IA_BF16)
    rc = launch_gated_norm_add<float, bf16_t>(h, delta, splits, stride, gate, gate_dtype, gate_stride, gate_splits, gstride, gate_bias, w,
                                              w_dtype, w_next, w_next_dtype, x, N, H, eps, stream);
  else
    return IA_ERR_BAD_ARG;
  if (rc != IA_OK) return rc;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// h[n, :] += table[index[n], :] (fp32 sums; the table in fp32 or bfloat16): a learned vector per position.  An index
// outside the table leaves NaN, never a stray read.
__global__ __launch_bounds__(256) void add_rows_kernel(float* __restrict__ h, const void* __restrict__ table, int dtype,
                                                       const int* __restrict__ index, int H, int rows) {
  const int n = blockIdx.x;
  const int r = index[n];
  float* hr = h + (size_t)n * H;
  if ((unsigned)r >= (unsigned)rows) {
    for (int i = threadIdx.x; i < H; i += 256) hr[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  for (int i = threadIdx.x; i < H; i += 256) hr[i] += load_as_float(table, dtype, (size_t)r * H + i);
}

extern "C" int ia_add_rows(float* h, const void* table, int dtype, const int* index, int N, int H, int rows,
                           hipStream_t stream) {
  if (N < 0 || H <= 0 || rows <= 0 || !h || !table || !index || (dtype != IA_F32 && dtype != IA_BF16)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  add_rows_kernel<<<N, 256, 0, stream>>>(h, table, dtype, index, H, rows);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_norm_add)
IA_OP(ia_gated_norm_add)
IA_OP(ia_add_rows)
