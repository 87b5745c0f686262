// Latent attention: keys and values of all heads are functions of one low-rank latent per token, and only the
// latent c [rank] and one rotated key part [rot] shared by all heads are cached.  With
//   score_h(i, j) = q_plain_h(i) . (U_h c_j) + q_rot_h(i) . k_rot(j)  =  (U_h^T q_plain_h(i)) . c_j + q_rot_h(i) . k_rot(j)
//   out_h(i)      = V_h sum_j p_h(i, j) c_j
// every head's query becomes a vector [rot | rank] against the one cached key [k_rot | c], and the value is the
// cached latent itself: attention with one key/value head of size rot + rank, which the attention kernels of this
// library serve as they are.  What is here is what stands around them:
//   ia_latent_prepare  from the projections' row [q heads (plain | rot) | latent | k_rot | ...] the row
//                      [H query heads (rot | .) | key (k_rot | c) | value (0 | c)] with c = RMSNorm(latent) * w;
//   ia_gemm_heads      a matrix product per head, out[n, h, :] = x[n, h, :] W_h^T (optionally times
//                      sigmoid(gate[n, h, :])): U_h^T on the plain query parts, V_h on the attended latents.
#include "common.h"
#include "tile_fma.h"

// One workgroup a token.  src row: [H * (dn + dr) | rank | dr | ...]; dst row: (H + 2) heads of d = dr + rank.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const T* __restrict__ src, int src_stride,
                                                             const T* __restrict__ lat_src, int lat_stride,
                                                             T* __restrict__ dst, int dst_stride,
                                                             const void* __restrict__ w, int w_dtype, int H, int dn,
                                                             int dr, int rank, float eps) {
  __shared__ float red[4];
  const int n = blockIdx.x, d = dr + rank;
  const T* s = src + (size_t)n * src_stride;
  T* o = dst + (size_t)n * dst_stride;
  for (int i = threadIdx.x; i < H * dr; i += 256) {          // the rotated query parts move to the heads' fronts
    const int h = i / dr, r = i - h * dr;
    o[(size_t)h * d + r] = s[(size_t)h * (dn + dr) + dn + r];
  }
  // the latent and the key's rotated part: behind the queries in their row, or rows of their own
  const T* lat = lat_src ? lat_src + (size_t)n * lat_stride : s + (size_t)H * (dn + dr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += 256) {
    const float v = to_float(lat[i]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  T* key = o + (size_t)H * d;
  T* val = key + d;
  for (int i = threadIdx.x; i < rank; i += 256) {
    const T c = from_float<T>(to_float(lat[i]) * inv * load_as_float(w, w_dtype, i));
    key[dr + i] = c;
    val[dr + i] = c;
  }
  for (int i = threadIdx.x; i < dr; i += 256) {
    key[i] = lat[rank + i];
    val[i] = from_float<T>(0.f);
  }
}

extern "C" int ia_latent_prepare(const void* src, int src_stride, const void* lat, int lat_stride, void* dst,
                                 int dst_stride, int dtype, const void* w, int w_dtype, int N, int H, int dn, int dr,
                                 int rank, float eps, hipStream_t stream) {
  if (N < 0 || H <= 0 || dn < 0 || dr < 0 || rank <= 0 || !(eps > 0.f) ||
      src_stride < H * (dn + dr) + (lat ? 0 : rank + dr) || (lat && lat_stride < rank + dr) ||
      dst_stride < (H + 2) * (dr + rank))
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (dtype == IA_F32)
    latent_prepare_kernel<float><<<N, 256, 0, stream>>>((const float*)src, src_stride, (const float*)lat, lat_stride, (float*)dst, dst_stride, w,
                                                        w_dtype, H, dn, dr, rank, eps);
  else if (dtype == IA_BF16)
    latent_prepare_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)src, src_stride, (const bf16_t*)lat, lat_stride, (bf16_t*)dst, dst_stride, w,
                                                         w_dtype, H, dn, dr, rank, eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// out[n, h, j] = (sum_k x[n, h, k] W[h, j, k]) * (gate ? sigmoid(gate[n, h * Nout + j]) : 1).
// grid: (tiles of Nout, tiles of N, H).  On the vector ALUs in fp32: the 32-bit path, and bfloat16 rows that
// cannot be read 16 bytes at a time.
template <typename T>
__global__ __launch_bounds__(256) void gemm_heads_kernel(const T* __restrict__ x, int x_row, int x_head,
                                                         const T* __restrict__ W, T* __restrict__ out, int o_row,
                                                         int o_head, const T* __restrict__ gate, int g_row, int N,
                                                         int Nout, int K) {
  __shared__ TileFmaLds lds;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * TF_T, n0 = blockIdx.x * TF_T;
  const int lr = threadIdx.x >> 2;
  const T* a_row = (m0 + lr < N) ? x + (size_t)(m0 + lr) * x_row + (size_t)h * x_head : nullptr;
  const T* w_row = (n0 + lr < Nout) ? W + ((size_t)h * Nout + n0 + lr) * K : nullptr;
  tile_64(a_row, w_row, K, lds, [&](int i, int j0, const float* v) {
    const int m = m0 + i;
    if (m >= N) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + j0 + j;
      if (c >= Nout) continue;
      float y = v[j];
      if (gate) {
        const float g = to_float(gate[(size_t)m * g_row + (size_t)h * Nout + c]);
        y = to_float(from_float<T>(y)) * (1.0f / (1.0f + expf(-g)));    // the product is stored first, as a tensor would be
      }
      out[(size_t)m * o_row + (size_t)h * o_head + c] = from_float<T>(y);
    }
  });
}

// The same on tiles of BM x 128 (tile_mfma_big): grid (tiles of 128 of Nout, tiles of BM of N, H).  With 2,048 rows
// tiles of 32 rows took 18 and 26 us where tiles of 128 took 30 and 28 (heads of 224 x 64 and 64 x 224).
template <int BM>
__global__ __launch_bounds__(256) void gemm_heads_big_kernel(const bf16_t* __restrict__ x, int x_row, int x_head,
                                                             const bf16_t* __restrict__ W, bf16_t* __restrict__ out,
                                                             int o_row, int o_head, const bf16_t* __restrict__ gate,
                                                             int g_row, int N, int Nout, int K) {
  __shared__ TileBigLds<BM> lds;
  const int h = blockIdx.z;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * TB_N;
  tile_mfma_big<BM>(
      [&](int r) { return x + (size_t)(m0 + r) * x_row + (size_t)h * x_head; },
      [&](int r) { return W + ((size_t)h * Nout + n0 + r) * K; }, N - m0, Nout - n0, K, lds,
      [&](int i, int j0, const float* v) {
        const int m = m0 + i;
        if (m >= N) return;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int c = n0 + j0 + j;
          if (c >= Nout) continue;
          float y = v[j];
          if (gate) {
            const float g = to_float(gate[(size_t)m * g_row + (size_t)h * Nout + c]);
            y = to_float(from_float<bf16_t>(y)) * (1.0f / (1.0f + expf(-g)));
          }
          out[(size_t)m * o_row + (size_t)h * o_head + c] = from_float<bf16_t>(y);
        }
      });
}

extern "C" int ia_gemm_heads(const void* x, int x_row, int x_head, const void* W, void* out, int o_row, int o_head,
                             const void* gate, int g_row, int dtype, int N, int H, int Nout, int K,
                             hipStream_t stream) {
  if (N < 0 || H <= 0 || Nout <= 0 || K <= 0 || x_head < 0 || o_head < 0 || x_row < (H - 1) * x_head + K ||
      o_row < (H - 1) * o_head + Nout || (gate && g_row < H * Nout))
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  dim3 grid((Nout + TF_T - 1) / TF_T, (N + TF_T - 1) / TF_T, H);
  if (grid.y > 65535u || grid.z > 65535u) return IA_ERR_UNSUPPORTED;
  if (dtype == IA_F32)
    gemm_heads_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_row, x_head, (const float*)W,
                                                              (float*)out, o_row, o_head, (const float*)gate, g_row,
                                                              N, Nout, K);
  else if (dtype == IA_BF16 && (K & 7) == 0 && tile_rows_aligned(x, x_row, x_head) && tile_rows_aligned(W, K)) {
    const int bm = 32;      // K is short here (a head's size): many small workgroups hide each other's few steps better than few large ones
    dim3 big((Nout + TB_N - 1) / TB_N, (N + bm - 1) / bm, H);
    if (big.y > 65535u) return IA_ERR_UNSUPPORTED;
    gemm_heads_big_kernel<32><<<big, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)W,
                                                       (bf16_t*)out, o_row, o_head, (const bf16_t*)gate, g_row, N,
                                                       Nout, K);
  }
  else if (dtype == IA_BF16)
    gemm_heads_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)W,
                                                               (bf16_t*)out, o_row, o_head, (const bf16_t*)gate, g_row,
                                                               N, Nout, K);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_latent_prepare)
IA_OP(ia_gemm_heads)
