// Routed experts: a token's feed-forward is the weighted sum of `top` small gated feed-forwards chosen among E.
//   ia_router_topk   z = logits + bias (fp32); the `top` largest (the lowest index among equals) and the softmax
//                    over those alone;
//   ia_moe_sort      the (token, choice) pairs grouped by expert: offsets[E + 1], perm[P];
//   ia_moe_gate_up   per expert, over its pairs' tokens: g = min(Wg x, limit), u = clamp(Wu x, -limit, limit),
//                    y = g sigmoid(alpha g) (u + 1); the rows of Wg and Wu alternate in the expert's matrix;
//   ia_moe_down      per expert: Wd y times the pair's routing weight, as fp32 into parts[choice, token, :], which
//                    the kernel that takes the feed-forward's result next adds in the order of the choices.
// Only the chosen experts' weights are read.  A pair's result is one chain of operations over its own token and
// its expert's weights, whatever else the step holds and wherever the sort has put it.
#include "common.h"
#include "tile_fma.h"

// One wave a token: lane l holds the logits of experts l, l + 64, ...; `top` rounds of "the largest not taken yet"
// (the lowest index among equals), each a maximum over the wave.
#define RT_PER_LANE 16        // experts a lane holds: E <= 64 * RT_PER_LANE
__global__ __launch_bounds__(256) void router_topk_kernel(const float* __restrict__ logits,
                                                          const void* __restrict__ bias, int bias_dtype,
                                                          int* __restrict__ ids, float* __restrict__ weights, int N,
                                                          int E, int top) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  const float* z = logits + (size_t)n * E;
  float v[RT_PER_LANE];
  unsigned taken = 0u;
#pragma unroll
  for (int c = 0; c < RT_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    v[c] = e < E ? z[e] + (bias ? load_as_float(bias, bias_dtype, e) : 0.f) : -INFINITY;
    if (e >= E) taken |= 1u << c;
  }
  float first_v = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best_v = -INFINITY;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int c = 0; c < RT_PER_LANE; ++c) {
      const bool free_ = !((taken >> c) & 1u);
      // a value that compares with nothing (NaN) counts as the smallest
      const float x = (v[c] == v[c]) ? v[c] : -INFINITY;
      if (free_ && (best_e == 0x7fffffff || x > best_v)) { best_v = x; best_e = lane + 64 * c; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best_v, o, IA_WAVE);
      const int oe = __shfl_xor(best_e, o, IA_WAVE);
      if (oe != 0x7fffffff && (best_e == 0x7fffffff || ov > best_v || (ov == best_v && oe < best_e))) {
        best_v = ov;
        best_e = oe;
      }
    }
    if ((best_e & 63) == lane) taken |= 1u << (best_e >> 6);
    if (k == 0) first_v = best_v;
    const float w = expf(best_v - first_v);
    sum += w;
    if (lane == 0) {
      ids[(size_t)n * top + k] = best_e;
      weights[(size_t)n * top + k] = w;
    }
  }
  const float inv = 1.0f / sum;
  if (lane == 0)
    for (int k = 0; k < top; ++k) weights[(size_t)n * top + k] *= inv;
}

extern "C" int ia_router_topk(const float* logits, const void* bias, int bias_dtype, int* ids, float* weights, int N,
                              int E, int top, hipStream_t stream) {
  if (N < 0 || E <= 0 || top <= 0 || top > E) return IA_ERR_BAD_ARG;
  if (E > 64 * RT_PER_LANE) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  router_topk_kernel<<<(N + 3) / 4, 256, 0, stream>>>(logits, bias, bias_dtype, ids, weights, N, E, top);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#define MOE_MAX_E 1024
// One workgroup.  offsets[e] .. offsets[e + 1] - 1 are the places in perm of expert e's pairs; the order of an
// expert's pairs is whatever the atomics give (no result depends on it).
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int* __restrict__ offsets,
                                                        int* __restrict__ perm, int P, int E) {
  __shared__ int cnt[MOE_MAX_E];
  __shared__ int cur[MOE_MAX_E];
  for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += 1024) {
    const int e = ids[p];
    if ((unsigned)e < (unsigned)E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = at;
      cur[e] = at;
      at += cnt[e];
    }
    offsets[E] = at;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += 1024) {
    const int e = ids[p];
    if ((unsigned)e < (unsigned)E) perm[atomicAdd(&cur[e], 1)] = p;
  }
}

extern "C" int ia_moe_sort(const int* ids, int* offsets, int* perm, int P, int E, hipStream_t stream) {
  if (P < 0 || E <= 0) return IA_ERR_BAD_ARG;
  if (E > MOE_MAX_E) return IA_ERR_UNSUPPORTED;
  moe_sort_kernel<<<1, 1024, 0, stream>>>(ids, offsets, perm, P, E);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// Tile t of the launch (`rows` pairs a tile, expert by expert): its expert and its first place in perm; false when
// the launch has more tiles than the step needs.
__device__ __forceinline__ bool moe_tile(const int* __restrict__ offsets, int E, int t, int& expert, int& first,
                                         int& last, int rows = TF_T) {
  int seen = 0;
  for (int e = 0; e < E; ++e) {
    const int lo = offsets[e], hi = offsets[e + 1];
    const int tiles = (hi - lo + rows - 1) / rows;
    if (t < seen + tiles) {
      expert = e;
      first = lo + (t - seen) * rows;
      last = hi;
      return true;
    }
    seen += tiles;
  }
  return false;
}

// grid: (tiles of 2 * ff columns, ceil(P / 64) + E).  Wgu [E, 2 ff, W]: row 2 j the gate's row j, row 2 j + 1 up's.
// On the vector ALUs in fp32: the 32-bit path, and bfloat16 rows that cannot be read 16 bytes at a time.
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ x, const T* __restrict__ Wgu,
                                                          T* __restrict__ y, const int* __restrict__ offsets,
                                                          const int* __restrict__ perm, int E, int top, int W,
                                                          int ff, float limit, float alpha) {
  __shared__ TileFmaLds lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last)) return;
  const int n0 = blockIdx.x * TF_T;
  const int lr = threadIdx.x >> 2;
  const T* a_row = (first + lr < last) ? x + (size_t)(perm[first + lr] / top) * W : nullptr;
  const T* w_row = (n0 + lr < 2 * ff) ? Wgu + ((size_t)e * 2 * ff + n0 + lr) * W : nullptr;
  tile_64(a_row, w_row, W, lds, [&](int i, int j0, const float* v) {
    const int p = first + i;
    if (p >= last) return;
#pragma unroll
    for (int j = 0; j < 4; j += 2) {
      const int c = n0 + j0 + j;
      if (c + 1 >= 2 * ff) continue;
      // both products are rounded as a stored tensor would be, then the activation in fp32
      const float g = fminf(to_float(from_float<T>(v[j])), limit);
      const float u = fminf(fmaxf(to_float(from_float<T>(v[j + 1])), -limit), limit);
      y[(size_t)p * ff + (c >> 1)] = from_float<T>(g * (1.0f / (1.0f + expf(-alpha * g))) * (u + 1.0f));
    }
  });
}

// The same on tiles of BM x BN (tile_mfma_big): grid (tiles of BN of the 2 ff columns, ceil(P / BM) + E).
template <int BM, int BN>
__global__ __launch_bounds__(BN == 256 ? 512 : 256) void moe_gate_up_big_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ Wgu,
                                                              bf16_t* __restrict__ y, const int* __restrict__ offsets,
                                                              const int* __restrict__ perm, int E, int top, int W,
                                                              int ff, float limit, float alpha) {
  __shared__ TileBigLds<BM, BN> lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last, BM)) return;
  const int n0 = blockIdx.x * BN;
  tile_mfma_big<BM, BN>(
      [&](int r) { return x + (size_t)(perm[first + r] / top) * W; },
      [&](int r) { return Wgu + ((size_t)e * 2 * ff + n0 + r) * W; }, last - first, 2 * ff - n0, W, lds,
      [&](int i, int j0, const float* v) {
        const int p = first + i;
        if (p >= last) return;
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
          const int c = n0 + j0 + j;
          if (c + 1 >= 2 * ff) continue;
          const float g = fminf(to_float(from_float<bf16_t>(v[j])), limit);
          const float u = fminf(fmaxf(to_float(from_float<bf16_t>(v[j + 1])), -limit), limit);
          y[(size_t)p * ff + (c >> 1)] = from_float<bf16_t>(g * (1.0f / (1.0f + expf(-alpha * g))) * (u + 1.0f));
        }
      });
}

// Rows a tile of the experts' products takes: 128 where an expert has some tens of pairs on average, else 32.
static inline int moe_tile_rows(int P, int E) { return (long)P >= 48L * E ? 128 : 32; }

extern "C" int ia_moe_gate_up(const void* x, const void* Wgu, void* y, const int* offsets, const int* perm, int dtype,
                              int P, int E, int top, int W, int ff, float limit, float alpha, hipStream_t stream) {
  if (P < 0 || E <= 0 || top <= 0 || W <= 0 || ff <= 0) return IA_ERR_BAD_ARG;
  if (P == 0) return IA_OK;
  dim3 grid((2 * ff + TF_T - 1) / TF_T, (P + TF_T - 1) / TF_T + E);
  if (grid.y > 65535u) return IA_ERR_UNSUPPORTED;
  if (dtype == IA_F32)
    moe_gate_up_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, (const float*)Wgu, (float*)y, offsets,
                                                               perm, E, top, W, ff, limit, alpha);
  else if (dtype == IA_BF16 && tile_rows_aligned(x, W) && tile_rows_aligned(Wgu, W)) {
    const int bm = moe_tile_rows(P, E);
    const int bn = bm == 128 ? 256 : TB_N;
    dim3 big((2 * ff + bn - 1) / bn, (P + bm - 1) / bm + E);
    if (big.y > 65535u) return IA_ERR_UNSUPPORTED;
    if (bm == 128)
      moe_gate_up_big_kernel<128, 256><<<big, 512, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wgu, (bf16_t*)y, offsets,
                                                           perm, E, top, W, ff, limit, alpha);
    else
      moe_gate_up_big_kernel<32, TB_N><<<big, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wgu, (bf16_t*)y, offsets,
                                                          perm, E, top, W, ff, limit, alpha);
  }
  else if (dtype == IA_BF16)
    moe_gate_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wgu, (bf16_t*)y,
                                                                offsets, perm, E, top, W, ff, limit, alpha);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// grid: (tiles of W columns, ceil(P / 64) + E).  Wd [E, W, ff]; parts [top, N, W] fp32.
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ y, const T* __restrict__ Wd,
                                                       float* __restrict__ parts, const float* __restrict__ weights,
                                                       const int* __restrict__ offsets, const int* __restrict__ perm,
                                                       int E, int top, int N, int W, int ff) {
  __shared__ TileFmaLds lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last)) return;
  const int n0 = blockIdx.x * TF_T;
  const int lr = threadIdx.x >> 2;
  const T* a_row = (first + lr < last) ? y + (size_t)(first + lr) * ff : nullptr;
  const T* w_row = (n0 + lr < W) ? Wd + ((size_t)e * W + n0 + lr) * ff : nullptr;
  tile_64(a_row, w_row, ff, lds, [&](int i, int j0, const float* v) {
    const int p = first + i;
    if (p >= last) return;
    const int pair = perm[p];
    const int token = pair / top, choice = pair - token * top;
    const float wt = weights[pair];
    float* o = parts + ((size_t)choice * N + token) * W;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + j0 + j;
      if (c < W) o[c] = to_float(from_float<T>(v[j])) * wt;
    }
  });
}

template <int BM, int BN>
__global__ __launch_bounds__(BN == 256 ? 512 : 256) void moe_down_big_kernel(const bf16_t* __restrict__ y, const bf16_t* __restrict__ Wd,
                                                           float* __restrict__ parts, const float* __restrict__ weights,
                                                           const int* __restrict__ offsets, const int* __restrict__ perm,
                                                           int E, int top, int N, int W, int ff) {
  __shared__ TileBigLds<BM, BN> lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last, BM)) return;
  const int n0 = blockIdx.x * BN;
  tile_mfma_big<BM, BN>(
      [&](int r) { return y + (size_t)(first + r) * ff; },
      [&](int r) { return Wd + ((size_t)e * W + n0 + r) * ff; }, last - first, W - n0, ff, lds,
      [&](int i, int j0, const float* v) {
        const int p = first + i;
        if (p >= last) return;
        const int pair = perm[p];
        const int token = pair / top, choice = pair - token * top;
        const float wt = weights[pair];
        float* o = parts + ((size_t)choice * N + token) * W;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int c = n0 + j0 + j;
          if (c < W) o[c] = to_float(from_float<bf16_t>(v[j])) * wt;
        }
      });
}

extern "C" int ia_moe_down(const void* y, const void* Wd, float* parts, const float* weights, const int* offsets,
                           const int* perm, int dtype, int N, int E, int top, int W, int ff, hipStream_t stream) {
  if (N < 0 || E <= 0 || top <= 0 || W <= 0 || ff <= 0) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  const int P = N * top;
  dim3 grid((W + TF_T - 1) / TF_T, (P + TF_T - 1) / TF_T + E);
  if (grid.y > 65535u) return IA_ERR_UNSUPPORTED;
  if (dtype == IA_F32)
    moe_down_kernel<float><<<grid, 256, 0, stream>>>((const float*)y, (const float*)Wd, parts, weights, offsets,
                                                            perm, E, top, N, W, ff);
  else if (dtype == IA_BF16 && tile_rows_aligned(y, ff) && tile_rows_aligned(Wd, ff)) {
    const int bm = moe_tile_rows(P, E);
    const int bn = bm == 128 ? 256 : TB_N;
    dim3 big((W + bn - 1) / bn, (P + bm - 1) / bm + E);
    if (big.y > 65535u) return IA_ERR_UNSUPPORTED;
    if (bm == 128)
      moe_down_big_kernel<128, 256><<<big, 512, 0, stream>>>((const bf16_t*)y, (const bf16_t*)Wd, parts, weights, offsets,
                                                        perm, E, top, N, W, ff);
    else
      moe_down_big_kernel<32, TB_N><<<big, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)Wd, parts, weights, offsets,
                                                       perm, E, top, N, W, ff);
  }
  else if (dtype == IA_BF16)
    moe_down_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)Wd, parts, weights,
                                                             offsets, perm, E, top, N, W, ff);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the experts of a step of many rows by the grouped form of the LDS-tiled product (ia_gemm_mfma_grouped) ----------
// The tokens' rows are first brought into the order of the sort (an expert's rows one after the other), the two
// products run expert by expert over those rows, and the activation and the routing weight are passes of their own:
//   ia_moe_gather   xs[p, :] = x[perm[p] / top, :]
//   ia_moe_glu      y[p, j] = g sigmoid(alpha g) (u + 1), g = min(gu[p, 2 j], limit), u = clamp(gu[p, 2 j + 1], +-limit)
//   ia_moe_scatter  parts[choice, token, :] = float(o[p, :]) * weights[perm[p]]
// All three in bfloat16 with rows that are read 16 bytes at a time.
__global__ __launch_bounds__(256) void moe_gather_kernel(const uint4* __restrict__ x, const int* __restrict__ perm,
                                                         uint4* __restrict__ xs, int top, int pieces) {
  const int p = blockIdx.x;
  const uint4* src = x + (size_t)(perm[p] / top) * pieces;
  uint4* dst = xs + (size_t)p * pieces;
  for (int i = threadIdx.x; i < pieces; i += 256) dst[i] = src[i];
}

extern "C" int ia_moe_gather(const void* x, const int* perm, void* xs, int P, int top, int W, hipStream_t stream) {
  if (P < 0 || top <= 0 || W <= 0) return IA_ERR_BAD_ARG;
  if ((W & 7) || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(xs)) & 15)) return IA_ERR_UNSUPPORTED;
  if (P == 0) return IA_OK;
  moe_gather_kernel<<<P, 256, 0, stream>>>((const uint4*)x, perm, (uint4*)xs, top, W / 8);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

__global__ __launch_bounds__(256) void moe_glu_kernel(const uint4* __restrict__ gu, uint2* __restrict__ y, size_t n4,
                                                      float limit, float alpha) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    const uint4 v = gu[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float g = fminf(__uint_as_float(w[k] << 16), limit);
      const float u = fminf(fmaxf(__uint_as_float(w[k] & 0xffff0000u), -limit), limit);
      o[k] = g * (1.0f / (1.0f + expf(-alpha * g))) * (u + 1.0f);
    }
    uint2 r;
    r.x = (uint32_t)float_to_bf16_bits(o[0]) | ((uint32_t)float_to_bf16_bits(o[1]) << 16);
    r.y = (uint32_t)float_to_bf16_bits(o[2]) | ((uint32_t)float_to_bf16_bits(o[3]) << 16);
    y[i] = r;
  }
}

extern "C" int ia_moe_glu(const void* gu, void* y, int P, int ff, float limit, float alpha, hipStream_t stream) {
  if (P < 0 || ff <= 0) return IA_ERR_BAD_ARG;
  if ((ff & 3) || ((reinterpret_cast<uintptr_t>(gu) | reinterpret_cast<uintptr_t>(y)) & 15)) return IA_ERR_UNSUPPORTED;
  const size_t n4 = (size_t)P * ff / 4;
  if (n4 == 0) return IA_OK;
  const unsigned grid = (unsigned)((n4 + 255) / 256 < 65536 ? (n4 + 255) / 256 : 65536);
  moe_glu_kernel<<<grid, 256, 0, stream>>>((const uint4*)gu, (uint2*)y, n4, limit, alpha);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

__global__ __launch_bounds__(256) void moe_scatter_kernel(const uint4* __restrict__ o, const int* __restrict__ perm,
                                                          const float* __restrict__ weights, float* __restrict__ parts,
                                                          int N, int top, int W) {
  const int p = blockIdx.x;
  const int pair = perm[p];
  const int token = pair / top, choice = pair - token * top;
  const float wt = weights[pair];
  const uint4* src = o + (size_t)p * (W / 8);
  float4* dst = reinterpret_cast<float4*>(parts + ((size_t)choice * N + token) * W);
  for (int i = threadIdx.x; i < W / 8; i += 256) {
    const uint4 v = src[i];
    dst[2 * i] = make_float4(__uint_as_float(v.x << 16) * wt, __uint_as_float(v.x & 0xffff0000u) * wt,
                             __uint_as_float(v.y << 16) * wt, __uint_as_float(v.y & 0xffff0000u) * wt);
    dst[2 * i + 1] = make_float4(__uint_as_float(v.z << 16) * wt, __uint_as_float(v.z & 0xffff0000u) * wt,
                                 __uint_as_float(v.w << 16) * wt, __uint_as_float(v.w & 0xffff0000u) * wt);
  }
}

extern "C" int ia_moe_scatter(const void* o, const int* perm, const float* weights, float* parts, int N, int top,
                              int W, hipStream_t stream) {
  if (N < 0 || top <= 0 || W <= 0) return IA_ERR_BAD_ARG;
  if ((W & 7) || ((reinterpret_cast<uintptr_t>(o) | reinterpret_cast<uintptr_t>(parts)) & 15)) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  moe_scatter_kernel<<<N * top, 256, 0, stream>>>((const uint4*)o, perm, weights, parts, N, top, W);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- experts without a gate, and a router whose choice and weights go by different numbers ----
//   ia_router_softmax_topk   s = softmax(z) over all experts; the `top` largest of s + correction are chosen (the
//                            lowest index among equals); the weights are the chosen s over their sum (+ 1e-20);
//   ia_moe_up                per expert, over its pairs' tokens: y = act(Wu x), Wu [E, ff, W]; act by the codes of
//                            ia_activation (2: the erf GELU, 3: the square of relu).
__device__ __forceinline__ float moe_act(float z, int act) {
  if (act == 3) { const float r = fmaxf(z, 0.f); return r * r; }
  if (act == 2) return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
  if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z;
}

__global__ __launch_bounds__(256) void router_softmax_topk_kernel(const float* __restrict__ logits,
                                                                  const void* __restrict__ corr, int corr_dtype,
                                                                  int* __restrict__ ids, float* __restrict__ weights,
                                                                  int N, int E, int top) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  const float* z = logits + (size_t)n * E;
  float s[RT_PER_LANE], v[RT_PER_LANE];
  unsigned taken = 0u;
  float zmax = -INFINITY;
#pragma unroll
  for (int c = 0; c < RT_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    s[c] = e < E ? z[e] : -INFINITY;
    zmax = fmaxf(zmax, s[c]);
    if (e >= E) taken |= 1u << c;
  }
  zmax = wave_max(zmax);
  float total = 0.f;
#pragma unroll
  for (int c = 0; c < RT_PER_LANE; ++c) {
    s[c] = (lane + 64 * c) < E ? expf(s[c] - zmax) : 0.f;
    total += s[c];
  }
  total = wave_sum(total);
  const float inv_total = 1.0f / total;
#pragma unroll
  for (int c = 0; c < RT_PER_LANE; ++c) {
    const int e = lane + 64 * c;
    s[c] *= inv_total;
    v[c] = e < E ? s[c] + (corr ? load_as_float(corr, corr_dtype, e) : 0.f) : -INFINITY;
  }
  float sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best_v = -INFINITY, best_s = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int c = 0; c < RT_PER_LANE; ++c) {
      const bool free_ = !((taken >> c) & 1u);
      const float x = (v[c] == v[c]) ? v[c] : -INFINITY;
      if (free_ && (best_e == 0x7fffffff || x > best_v)) { best_v = x; best_e = lane + 64 * c; best_s = s[c]; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best_v, o, IA_WAVE), os = __shfl_xor(best_s, o, IA_WAVE);
      const int oe = __shfl_xor(best_e, o, IA_WAVE);
      if (oe != 0x7fffffff && (best_e == 0x7fffffff || ov > best_v || (ov == best_v && oe < best_e))) {
        best_v = ov;
        best_e = oe;
        best_s = os;
      }
    }
    if ((best_e & 63) == lane) taken |= 1u << (best_e >> 6);
    sum += best_s;
    if (lane == 0) {
      ids[(size_t)n * top + k] = best_e;
      weights[(size_t)n * top + k] = best_s;
    }
  }
  const float inv = 1.0f / (sum + 1e-20f);
  if (lane == 0)
    for (int k = 0; k < top; ++k) weights[(size_t)n * top + k] *= inv;
}

extern "C" int ia_router_softmax_topk(const float* logits, const void* corr, int corr_dtype, int* ids, float* weights,
                                      int N, int E, int top, hipStream_t stream) {
  if (N < 0 || E <= 0 || top <= 0 || top > E || !logits || !ids || !weights) return IA_ERR_BAD_ARG;
  if (E > 64 * RT_PER_LANE) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  router_softmax_topk_kernel<<<(N + 3) / 4, 256, 0, stream>>>(logits, corr, corr_dtype, ids, weights, N, E, top);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(const T* __restrict__ x, const T* __restrict__ Wu, T* __restrict__ y,
                                                     const int* __restrict__ offsets, const int* __restrict__ perm,
                                                     int E, int top, int W, int ff, int act) {
  __shared__ TileFmaLds lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last)) return;
  const int n0 = blockIdx.x * TF_T;
  const int lr = threadIdx.x >> 2;
  const T* a_row = (first + lr < last) ? x + (size_t)(perm[first + lr] / top) * W : nullptr;
  const T* w_row = (n0 + lr < ff) ? Wu + ((size_t)e * ff + n0 + lr) * W : nullptr;
  tile_64(a_row, w_row, W, lds, [&](int i, int j0, const float* v) {
    const int p = first + i;
    if (p >= last) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + j0 + j;
      // the product is rounded as a stored tensor would be, then the activation in fp32
      if (c < ff) y[(size_t)p * ff + c] = from_float<T>(moe_act(to_float(from_float<T>(v[j])), act));
    }
  });
}

template <int BM, int BN>
__global__ __launch_bounds__(BN == 256 ? 512 : 256) void moe_up_big_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ Wu,
                                                              bf16_t* __restrict__ y, const int* __restrict__ offsets,
                                                              const int* __restrict__ perm, int E, int top, int W,
                                                              int ff, int act) {
  __shared__ TileBigLds<BM, BN> lds;
  int e, first, last;
  if (!moe_tile(offsets, E, blockIdx.y, e, first, last, BM)) return;
  const int n0 = blockIdx.x * BN;
  tile_mfma_big<BM, BN>(
      [&](int r) { return x + (size_t)(perm[first + r] / top) * W; },
      [&](int r) { return Wu + ((size_t)e * ff + n0 + r) * W; }, last - first, ff - n0, W, lds,
      [&](int i, int j0, const float* v) {
        const int p = first + i;
        if (p >= last) return;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int c = n0 + j0 + j;
          if (c < ff) y[(size_t)p * ff + c] = from_float<bf16_t>(moe_act(to_float(from_float<bf16_t>(v[j])), act));
        }
      });
}

extern "C" int ia_moe_up(const void* x, const void* Wu, void* y, const int* offsets, const int* perm, int dtype, int P,
                         int E, int top, int W, int ff, int act, hipStream_t stream) {
  if (P < 0 || E <= 0 || top <= 0 || W <= 0 || ff <= 0 || act < 0 || act > 3) return IA_ERR_BAD_ARG;
  if (P == 0) return IA_OK;
  dim3 grid((ff + TF_T - 1) / TF_T, (P + TF_T - 1) / TF_T + E);
  if (grid.y > 65535u) return IA_ERR_UNSUPPORTED;
  if (dtype == IA_F32)
    moe_up_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, (const float*)Wu, (float*)y, offsets, perm, E, top,
                                                   W, ff, act);
  else if (dtype == IA_BF16 && tile_rows_aligned(x, W) && tile_rows_aligned(Wu, W)) {
    const int bm = moe_tile_rows(P, E);
    const int bn = bm == 128 ? 256 : TB_N;
    dim3 big((ff + bn - 1) / bn, (P + bm - 1) / bm + E);
    if (big.y > 65535u) return IA_ERR_UNSUPPORTED;
    if (bm == 128)
      moe_up_big_kernel<128, 256><<<big, 512, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wu, (bf16_t*)y, offsets, perm,
                                                           E, top, W, ff, act);
    else
      moe_up_big_kernel<32, TB_N><<<big, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wu, (bf16_t*)y, offsets, perm,
                                                          E, top, W, ff, act);
  } else if (dtype == IA_BF16)
    moe_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)Wu, (bf16_t*)y, offsets, perm, E,
                                                    top, W, ff, act);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_router_topk)
IA_OP(ia_moe_sort)
IA_OP(ia_moe_gate_up)
IA_OP(ia_moe_down)
IA_OP(ia_moe_gather)
IA_OP(ia_moe_glu)
IA_OP(ia_moe_scatter)
IA_OP(ia_router_softmax_topk)
IA_OP(ia_moe_up)
