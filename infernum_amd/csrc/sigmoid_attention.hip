// Attention whose weights are sigmoids, not a softmax: for the query of head h at position i and the key at j <= i,
//     w_ij = sigmoid( scale q_i.k_j - r1_h ln(1 + r2_h (i - j)) + b_h ),      o_i = g_ih sum_j w_ij v_j,
// nothing normalised over the keys, g = sigmoid(gate logit) one number per token and head.  Query heads share
// key/value heads in groups; keys have `dim` values, values `vdim`.
//
//   ia_sigattn_prepare   from a token's projected row [q | k | v | ...]: biases, the root mean square over ALL of a
//                        row's queries (and over all of its keys) with a weight per value, the query's factor
//                        1 + coef ln(floor((p + 1) / every) + 1), queries into their own rows, keys and values into
//                        their pages;
//   ia_sigattn_generic   one wave per (token, head), fp32 throughout, keys 64 at a time in the order of their
//                        positions: the 32-bit path and the plain twin of the matrix-core kernels;
//   ia_sigattn_mfma      bf16 on the matrix cores: single tokens (the query heads of a key/value head side by side,
//                        the keys in parts over workgroups and waves, joined in a fixed order) and portions of
//                        prompts (a wave per 16 rows of a head).
//
// Pages: keys [num_pages, nkv, page_size, dim], values transposed [num_pages, nkv, vdim, page_size] (four keys of
// one value channel are 8 contiguous bytes, the operand of the second product); block_tables[s, j / page_size]
// is the page of key j of request s.  A sum of weights has no reference point to move, so parts of the keys add up.
#include "common.h"

#define SA_MAX_D 640

template <typename T>
__global__ __launch_bounds__(256) void sigattn_prepare_kernel(
    const T* __restrict__ proj, int proj_stride, const float* __restrict__ bq, const float* __restrict__ bk,
    const float* __restrict__ bv, const float* __restrict__ wq, const float* __restrict__ wk, float eps, float temp_coef,
    int temp_every, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ q_out,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int dim, int vdim, int page_size, int num_pages) {
  __shared__ float red[4];
  const int n = blockIdx.x, tid = threadIdx.x;
  const T* row = proj + (size_t)n * proj_stride;
  const int nq = nh * dim, nk = nkv * dim, nv = nkv * vdim;
  float ss = 0.f;
  for (int i = tid; i < nq; i += 256) {
    const float x = to_float(row[i]) + (bq ? bq[i] : 0.f);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum<256>(ss, red);
  float f = 1.0f / sqrtf(ss / (float)nq + eps);
  if (temp_every > 0) f *= 1.0f + temp_coef * logf((float)((positions[n] + 1) / temp_every) + 1.0f);
  for (int i = tid; i < nq; i += 256) {
    const float x = to_float(row[i]) + (bq ? bq[i] : 0.f);
    q_out[(size_t)n * nq + i] = from_float<T>(x * f * wq[i]);
  }
  if (!slots) return;
  const int slot = slots[n];
  const int page = slot / page_size, off = slot - page * page_size;
  if ((unsigned)page >= (unsigned)num_pages) return;          // a token without a place: nothing is written
  float sk = 0.f;
  for (int i = tid; i < nk; i += 256) {
    const float x = to_float(row[nq + i]) + (bk ? bk[i] : 0.f);
    sk = fmaf(x, x, sk);
  }
  sk = block_sum<256>(sk, red);
  const float fk = 1.0f / sqrtf(sk / (float)nk + eps);
  for (int i = tid; i < nk; i += 256) {
    const int g = i / dim, c = i - g * dim;
    const float x = to_float(row[nq + i]) + (bk ? bk[i] : 0.f);
    k_pages[(((size_t)page * nkv + g) * page_size + off) * dim + c] = from_float<T>(x * fk * wk[i]);
  }
  for (int i = tid; i < nv; i += 256) {
    const int g = i / vdim, c = i - g * vdim;
    const float x = to_float(row[nq + nk + i]) + (bv ? bv[i] : 0.f);
    v_pages[(((size_t)page * nkv + g) * vdim + c) * page_size + off] = from_float<T>(x);
  }
}

// proj rows [nh dim | nkv dim | nkv vdim | ...] of proj_stride values; biases and norm weights fp32 (biases nullable);
// temp_every 0: no factor on the queries; slots null: queries only (the pages are another run's).
extern "C" int ia_sigattn_prepare(const void* proj, int code, int proj_stride, const float* bq, const float* bk,
                                  const float* bv, const float* wq, const float* wk, float eps, float temp_coef,
                                  int temp_every, const int* positions, const int* slots, void* q_out, void* k_pages,
                                  void* v_pages, int N, int nh, int nkv, int dim, int vdim, int page_size, int num_pages,
                                  hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || dim <= 0 || vdim <= 0 || !(eps > 0.f) || temp_every < 0 ||
      proj_stride < nh * dim + (slots ? nkv * (dim + vdim) : 0))
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!proj || !wq || !q_out || !positions || (slots && (!wk || !k_pages || !v_pages || page_size <= 0 || num_pages <= 0)))
    return IA_ERR_BAD_ARG;
  if (code == IA_F32)
    sigattn_prepare_kernel<float><<<N, 256, 0, stream>>>((const float*)proj, proj_stride, bq, bk, bv, wq, wk, eps,
                                                         temp_coef, temp_every, positions, slots, (float*)q_out,
                                                         (float*)k_pages, (float*)v_pages, nh, nkv, dim, vdim, page_size,
                                                         num_pages);
  else if (code == IA_BF16)
    sigattn_prepare_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)proj, proj_stride, bq, bk, bv, wq, wk, eps,
                                                          temp_coef, temp_every, positions, slots, (bf16_t*)q_out,
                                                          (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv, dim, vdim,
                                                          page_size, num_pages);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

template <typename T>
__global__ __launch_bounds__(64) void sigattn_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const T* __restrict__ gate, int gate_stride, T* __restrict__ out, const int* __restrict__ token_seq,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int bt_stride, const float* __restrict__ r1,
    const float* __restrict__ r2, const float* __restrict__ pb, int nh, int nkv, int dim, int vdim, int page_size,
    int num_pages, float scale) {
  __shared__ float qs[SA_MAX_D];
  __shared__ float ps[64];
  __shared__ int rs[64];
  __shared__ size_t vs[64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[n];
  const int pos = positions[n];
  const int g = h / (nh / nkv);
  const int* bt = block_tables + (size_t)s * bt_stride;
  const T* qr = q + (size_t)n * q_stride + (size_t)h * dim;
  for (int i = lane; i < dim; i += 64) qs[i] = to_float(qr[i]);
  __syncthreads();
  const float a1 = r1 ? r1[h] : 0.f, a2 = r2 ? r2[h] : 0.f, b = pb ? pb[h] : 0.f;
  float acc[SA_MAX_D / 64];
#pragma unroll
  for (int c = 0; c < SA_MAX_D / 64; ++c) acc[c] = 0.f;
  for (int j0 = 0; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    float p = 0.f;
    int row = 0;
    size_t vat = 0;
    if (j <= pos) {
      const int page = bt[j / page_size];
      if ((unsigned)page < (unsigned)num_pages) {
        row = (page * nkv + g) * page_size + (j % page_size);
        vat = ((size_t)page * nkv + g) * vdim * page_size + (j % page_size);
        const T* kr = k_pages + (size_t)row * dim;
        float dot = 0.f;
        for (int i = 0; i < dim; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
        const float sc = dot * scale - a1 * log1pf(a2 * (float)(pos - j)) + b;
        p = 1.0f / (1.0f + expf(-sc));
      } else {
        p = __uint_as_float(0x7fc00000u);     // a block table without a page here: poison, never a stray read
      }
    }
    ps[lane] = p;
    rs[lane] = row;
    vs[lane] = vat;
    __syncthreads();
    const int cnt = (pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64;
    for (int jj = 0; jj < cnt; ++jj) {
      const T* vr = v_pages + vs[jj];
      const float pj = ps[jj];
#pragma unroll
      for (int c = 0; c < SA_MAX_D / 64; ++c) {
        const int i = lane + 64 * c;
        if (i < vdim) acc[c] = fmaf(pj, to_float(vr[(size_t)i * page_size]), acc[c]);
      }
    }
    __syncthreads();
  }
  float gt = 1.0f;
  if (gate) gt = 1.0f / (1.0f + expf(-to_float(gate[(size_t)n * gate_stride + h])));
  T* o = out + ((size_t)n * nh + h) * vdim;
#pragma unroll
  for (int c = 0; c < SA_MAX_D / 64; ++c) {
    const int i = lane + 64 * c;
    if (i < vdim) o[i] = from_float<T>(acc[c] * gt);
  }
}

// q rows of q_stride values (head h's dim values from h * dim); gate (nullable): rows of gate_stride values, head h's
// logit at [h]; r1, r2, pb (nullable) fp32 [nh]; out [N, nh vdim].
extern "C" int ia_sigattn_generic(const void* q, int q_stride, const void* k_pages, const void* v_pages, const void* gate,
                                  int gate_stride, void* out, int dtype, const int* token_seq, const int* positions,
                                  const int* block_tables, int bt_stride, const float* r1, const float* r2,
                                  const float* pb, int N, int nh, int nkv, int dim, int vdim, int page_size,
                                  int num_pages, float scale, hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || dim <= 0 || dim > SA_MAX_D || vdim <= 0 || vdim > SA_MAX_D ||
      page_size <= 0 || num_pages <= 0 || bt_stride <= 0 || q_stride < nh * dim || (gate && gate_stride < nh))
    return IA_ERR_BAD_ARG;
  if (nh > 65535) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  dim3 grid(N, nh);
  if (dtype == IA_F32)
    sigattn_generic_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_stride, (const float*)k_pages,
                                                           (const float*)v_pages, (const float*)gate, gate_stride,
                                                           (float*)out, token_seq, positions, block_tables, bt_stride,
                                                           r1, r2, pb, nh, nkv, dim, vdim, page_size, num_pages, scale);
  else if (dtype == IA_BF16)
    sigattn_generic_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_pages,
                                                            (const bf16_t*)v_pages, (const bf16_t*)gate, gate_stride,
                                                            (bf16_t*)out, token_seq, positions, block_tables, bt_stride,
                                                            r1, r2, pb, nh, nkv, dim, vdim, page_size, num_pages, scale);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_sigattn_prepare)
IA_OP(ia_sigattn_generic)
