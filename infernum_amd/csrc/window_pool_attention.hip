// Attention over a sliding window of single keys and, before the window, whole blocks of keys that are seen through
// their means; key and value heads of different sizes; an optional sink per head in the softmax's denominator.
//
// A query at position p sees the keys j with 0 <= p - j < window (window 0: every j <= p), and, with blocks of P
// positions (block b holds b P .. b P + P - 1), every block whose last position is at most p - window: the block's
// key is the mean of its P keys as the pages hold them, its value the mean of its P values.  Blocks and keys share
// one softmax.  A sink s_h adds exp(s_h) to the denominator and nothing to the sum.
//
//   ia_wpa_prepare     from a token's projected row [nh q heads of d | nkv k heads of d | nkv v heads of dv]: biases,
//                      rotation of the first `rot` values of every q and k head (value i with value i + rot/2),
//                      then every q and k head divided by its root mean square; queries to q_out, keys and values
//                      to their pages.
//   ia_wpa_pool        for every token of the step that is the last of its block: the means of the block's keys and
//                      values, read from the pages, into the pooled pages.
//   ia_wpa_attention   a wave per (token, query head): blocks first, then the window's keys, 64 at a time, in the
//                      order of their positions, so that a position's result does not depend on the batch.
//   ia_rms_rows        y = x / sqrt(mean(x^2) + eps) * w over C values of every row (w nullable).
//   ia_gelu_mul_rows   y[n, j] = gelu_tanh(u[n, j]) * table[ids[n], col0 + j].
//
// Token pages: keys [num_pages, nkv, page_size, d], values transposed within the page, [num_pages, nkv, dv, page_size]
// (what the matrix-core kernels of window_pool_attention_mfma.hip read 8 bytes at a time).  Pooled pages:
// [num_pages, nkv, E, d] and [.., E, dv] with E = (page_size - 1) / P + 1 entries a page: block b lies in the page of
// its last position t = b P + P - 1, at entry (t % page_size) / P.  The token pages and the pooled pages have block
// tables of their own (the token pages may be given back once the window and the open block have passed them).
// All arithmetic is fp32.
#include "common.h"

#define WPA_MAX_D 640
#define WPA_POOL_CHUNK 512      // positions of a block whose places are looked up together

template <typename T>
__global__ __launch_bounds__(64) void wpa_prepare_kernel(
    const T* __restrict__ src, int src_stride, const float* __restrict__ bias, T* __restrict__ q_out, int q_stride,
    const int* __restrict__ positions, const int* __restrict__ slots, const void* __restrict__ freq, int freq_f64,
    int rot, int unit_norm, float eps, T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int d, int dv,
    int ps, int num_pages) {
  __shared__ float x[WPA_MAX_D];
  const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const bool is_v = head >= nh + nkv, is_k = !is_v && head >= nh;
  const int size = is_v ? dv : d;
  const int col = is_v ? (nh + nkv) * d + (head - nh - nkv) * dv : head * d;
  const T* s = src + (size_t)n * src_stride + col;
  for (int i = lane; i < size; i += 64) x[i] = to_float(s[i]) + (bias ? bias[col + i] : 0.f);
  __syncthreads();
  T* dst;
  size_t step = 1;               // from a value to the next where it is written
  if (!is_v) {
    const int half = rot >> 1, pos = positions[n];
    for (int i = lane; i < half; i += 64) {
      float sn, cs, lo, hi;
      rope_sincos(pos, freq, freq_f64, i, sn, cs);
      rope_pair(x[i], x[i + half], cs, sn, lo, hi);
      x[i] = lo;
      x[i + half] = hi;
    }
    __syncthreads();
    if (unit_norm) {
      float ss = 0.f;
      for (int i = lane; i < d; i += 64) ss = fmaf(x[i], x[i], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)d + eps);
      for (int i = lane; i < d; i += 64) x[i] *= inv;
      __syncthreads();
    }
  }
  if (!is_k && !is_v) {
    dst = q_out + (size_t)n * q_stride + (size_t)head * d;
  } else {
    const int slot = slots[n], page = slot / ps, off = slot - page * ps;
    if ((unsigned)page >= (unsigned)num_pages) return;
    if (is_k) dst = k_pages + (((size_t)page * nkv + (head - nh)) * ps + off) * d;
    else {
      dst = v_pages + ((size_t)page * nkv + (head - nh - nkv)) * dv * ps + off;
      step = (size_t)ps;
    }
  }
  for (int i = lane; i < size; i += 64) dst[i * step] = from_float<T>(x[i]);
}

extern "C" int ia_wpa_prepare(const void* src, int src_stride, const float* bias, void* q_out, int q_stride, int dtype,
                              const int* positions, const int* slots, const void* freq, int freq_f64, int rot,
                              int unit_norm, float eps, void* k_pages, void* v_pages, int N, int nh, int nkv, int d,
                              int dv, int ps, int num_pages, hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || d <= 0 || dv <= 0 || d > WPA_MAX_D || dv > WPA_MAX_D || rot < 0 || rot > d ||
      (rot & 1) || ps <= 0 || num_pages <= 0 || src_stride < (nh + nkv) * d + nkv * dv || q_stride < nh * d)
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!src || !q_out || !positions || !slots || !k_pages || !v_pages || (rot && !freq)) return IA_ERR_BAD_ARG;
  if (nh + 2 * nkv > 65535) return IA_ERR_UNSUPPORTED;
  dim3 grid(N, nh + 2 * nkv);
  if (dtype == IA_F32)
    wpa_prepare_kernel<float><<<grid, 64, 0, stream>>>((const float*)src, src_stride, bias, (float*)q_out, q_stride,
                                                       positions, slots, freq, freq_f64, rot, unit_norm, eps,
                                                       (float*)k_pages, (float*)v_pages, nh, nkv, d, dv, ps, num_pages);
  else if (dtype == IA_BF16)
    wpa_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)src, src_stride, bias, (bf16_t*)q_out, q_stride,
                                                        positions, slots, freq, freq_f64, rot, unit_norm, eps,
                                                        (bf16_t*)k_pages, (bf16_t*)v_pages, nh, nkv, d, dv, ps,
                                                        num_pages);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// grid (N, nkv), 256 threads: a thread a value of the block's key or value, the block's positions added in their
// order (the loads of sixteen are in flight together).  A token that is not the last of its block leaves at once.
template <typename T>
__global__ __launch_bounds__(256) void wpa_pool_kernel(const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                                                       T* __restrict__ pk_pages, T* __restrict__ pv_pages,
                                                       const int* __restrict__ token_seq,
                                                       const int* __restrict__ positions, const int* __restrict__ bt_tok,
                                                       int bt_tok_stride, const int* __restrict__ bt_pool,
                                                       int bt_pool_stride, int nkv, int d, int dv, int ps, int num_pages,
                                                       int num_pool_pages, int P, int N, int stride) {
  // The tokens that close a block stand P apart; workgroups go to dies and compute units by their number in turn,
  // so with tokens in the order of the workgroups a block size that is a power of two (as those turns are) sends all
  // the work to a few compute units (blocks of 64 in a prompt of 2,048: 66 us against under 15 for blocks of 7).  The
  // tokens are dealt out in steps of a prime modulo an ODD number of workgroups instead (N or N + 1; the one too many
  // leaves): steps modulo a power of two would keep the tokens' remainders by powers of two together.
  const int modulus = (int)gridDim.x;
  const int n = (int)(((long long)blockIdx.x * stride) % modulus), g = blockIdx.y;
  if (n >= N) return;
  const int pos = positions[n];
  if ((pos + 1) % P != 0) return;
  const int s = token_seq[n];
  const int* bt = bt_tok + (size_t)s * bt_tok_stride;
  const int E = (ps - 1) / P + 1;
  const int ppage = bt_pool[(size_t)s * bt_pool_stride + pos / ps];
  if ((unsigned)ppage >= (unsigned)num_pool_pages) return;
  const int entry = (pos % ps) / P;
  T* pk = pk_pages + (((size_t)ppage * nkv + g) * E + entry) * d;
  T* pv = pv_pages + (((size_t)ppage * nkv + g) * E + entry) * dv;
  const float inv = 1.0f / (float)P;
  // where each of the block's positions lies, found once for all values: the sums' loads then wait for nothing
  __shared__ int s_page[WPA_POOL_CHUNK], s_off[WPA_POOL_CHUNK];
  __shared__ int s_bad;
  if (threadIdx.x == 0) s_bad = 0;
  float acc[(WPA_MAX_D * 2 + 255) / 256];
#pragma unroll
  for (int u = 0; u < (WPA_MAX_D * 2 + 255) / 256; ++u) acc[u] = 0.f;
  for (int j0 = pos - P + 1; j0 <= pos; j0 += WPA_POOL_CHUNK) {
    const int cnt = pos - j0 + 1 < WPA_POOL_CHUNK ? pos - j0 + 1 : WPA_POOL_CHUNK;
    __syncthreads();
    for (int t = threadIdx.x; t < cnt; t += 256) {
      const int j = j0 + t, page = bt[j / ps];
      const bool ok = (unsigned)page < (unsigned)num_pages;
      if (!ok) s_bad = 1;
      s_page[t] = ok ? page : 0;
      s_off[t] = j % ps;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < (WPA_MAX_D * 2 + 255) / 256; ++u) {
      const int i = threadIdx.x + 256 * u;
      if (i >= d + dv) break;
      const bool key = i < d;
      const int c = key ? i : i - d;
      float a = acc[u];
      for (int t = 0; t < cnt; t += 16) {                 // sixteen loads are out before the first is added
        float x[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int tt = t + e < cnt ? t + e : cnt - 1;
          const size_t head_page = (size_t)s_page[tt] * nkv + g;
          // one load from a chosen address, not a choice between two loads: nothing waits between the sixteen
          const T* at = key ? k_pages + (head_page * ps + s_off[tt]) * d + c : v_pages + (head_page * dv + c) * ps + s_off[tt];
          x[e] = to_float(*at);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) a += t + e < cnt ? x[e] : 0.f;      // in the order of the positions
      }
      acc[u] = a;
    }
  }
  __syncthreads();
  const bool bad = s_bad != 0;                             // a key of the block has no page: poison, never a stray read
#pragma unroll
  for (int u = 0; u < (WPA_MAX_D * 2 + 255) / 256; ++u) {
    const int i = threadIdx.x + 256 * u;
    if (i >= d + dv) break;
    const float r = bad ? __uint_as_float(0x7fc00000u) : acc[u] * inv;
    if (i < d) pk[i] = from_float<T>(r);
    else pv[i - d] = from_float<T>(r);
  }
}

extern "C" int ia_wpa_pool(const void* k_pages, const void* v_pages, void* pk_pages, void* pv_pages, int dtype,
                           const int* token_seq, const int* positions, const int* bt_tok, int bt_tok_stride,
                           const int* bt_pool, int bt_pool_stride, int N, int nkv, int d, int dv, int ps, int num_pages,
                           int num_pool_pages, int P, hipStream_t stream) {
  if (N < 0 || nkv <= 0 || d <= 0 || dv <= 0 || ps <= 0 || num_pages <= 0 || num_pool_pages <= 0 || P <= 0 ||
      bt_tok_stride <= 0 || bt_pool_stride <= 0 || nkv > 65535)
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!k_pages || !v_pages || !pk_pages || !pv_pages || !token_seq || !positions || !bt_tok || !bt_pool)
    return IA_ERR_BAD_ARG;
  const int modulus = N | 1;
  dim3 grid(modulus, nkv);
  int stride = 1;
  for (int prime : {7919, 104729, 1299709})
    if (modulus % prime != 0) { stride = prime; break; }
  if (dtype == IA_F32)
    wpa_pool_kernel<float><<<grid, 256, 0, stream>>>((const float*)k_pages, (const float*)v_pages, (float*)pk_pages,
                                                    (float*)pv_pages, token_seq, positions, bt_tok, bt_tok_stride,
                                                    bt_pool, bt_pool_stride, nkv, d, dv, ps, num_pages, num_pool_pages, P,
                                                    N, stride);
  else if (dtype == IA_BF16)
    wpa_pool_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)pk_pages,
                                                     (bf16_t*)pv_pages, token_seq, positions, bt_tok, bt_tok_stride,
                                                     bt_pool, bt_pool_stride, nkv, d, dv, ps, num_pages, num_pool_pages,
                                                     P, N, stride);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// One stretch of up to 64 keys (or blocks): lane `lane` holds the key at row `row` of its pool when `valid`;
// `ok` false: the key is needed and has no page.  Updates the running maximum, denominator and sums.
// ``row``: the key's row in its pool; ``vat``: where the key's first value stands, ``vstep`` from a value to the next.
template <typename T>
__device__ __forceinline__ void wpa_round(const float* qs, const T* __restrict__ kp, const T* __restrict__ vp, bool valid,
                                          bool ok, size_t row, size_t vat, size_t vstep, int cnt, int d, int dv,
                                          float scale, float& m, float& l, float* acc, float* ps_, size_t* rs_) {
  const int lane = threadIdx.x;
  float sc = -INFINITY;
  if (valid) {
    if (ok) {
      const T* kr = kp + row * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
      sc = dot * scale;
    } else {
      sc = __uint_as_float(0x7fc00000u);
    }
  }
  const float m_new = fmaxf(m, wave_max(sc));
  const float p = valid ? expf(sc - m_new) : 0.f;
  const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
  l = l * corr + wave_sum(p);
#pragma unroll
  for (int c = 0; c < WPA_MAX_D / 64; ++c) acc[c] *= corr;
  ps_[lane] = p;
  rs_[lane] = ok ? vat : 0;
  __syncthreads();
  for (int jj = 0; jj < cnt; ++jj) {
    const T* vr = vp + rs_[jj];
    const float pj = ps_[jj];
#pragma unroll
    for (int c = 0; c < WPA_MAX_D / 64; ++c) {
      const int dim = lane + 64 * c;
      if (dim < dv) acc[c] = fmaf(pj, to_float(vr[(size_t)dim * vstep]), acc[c]);
    }
  }
  __syncthreads();
  m = m_new;
}

template <typename T>
__global__ __launch_bounds__(64) void wpa_attention_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const T* __restrict__ pk_pages, const T* __restrict__ pv_pages, T* __restrict__ out, int out_stride,
    const float* __restrict__ sinks, const int* __restrict__ token_seq, const int* __restrict__ positions,
    const int* __restrict__ bt_tok, int bt_tok_stride, const int* __restrict__ bt_pool, int bt_pool_stride, int nh,
    int nkv, int d, int dv, int ps, int num_pages, int num_pool_pages, float scale, int window, int P) {
  __shared__ float qs[WPA_MAX_D];
  __shared__ float ps_[64];
  __shared__ size_t rs_[64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[n], pos = positions[n];
  const int g = h / (nh / nkv);
  const T* qr = q + (size_t)n * q_stride + (size_t)h * d;
  for (int i = lane; i < d; i += 64) qs[i] = to_float(qr[i]);
  __syncthreads();
  float m = -INFINITY, l = 0.f;
  float acc[WPA_MAX_D / 64];
#pragma unroll
  for (int c = 0; c < WPA_MAX_D / 64; ++c) acc[c] = 0.f;
  // the blocks that lie wholly before the window
  if (window > 0 && P > 0 && pos - window + 1 >= P) {
    const int nb = (pos - window + 1) / P;
    const int E = (ps - 1) / P + 1;
    const int* bt = bt_pool + (size_t)s * bt_pool_stride;
    for (int b0 = 0; b0 < nb; b0 += 64) {
      const int b = b0 + lane;
      const bool valid = b < nb;
      bool ok = false;
      size_t row = 0;
      if (valid) {
        const int t = b * P + P - 1;
        const int page = bt[t / ps];
        ok = (unsigned)page < (unsigned)num_pool_pages;
        if (ok) row = ((size_t)page * nkv + g) * E + (t % ps) / P;
      }
      wpa_round<T>(qs, pk_pages, pv_pages, valid, ok, row, row * dv, 1, (nb - b0) < 64 ? (nb - b0) : 64, d, dv, scale, m,
                   l, acc, ps_, rs_);
    }
  }
  // the window's keys
  {
    const int j_lo = ia_first_visible_key(pos, window > 0 ? window : 0);
    const int* bt = bt_tok + (size_t)s * bt_tok_stride;
    for (int j0 = j_lo; j0 <= pos; j0 += 64) {
      const int j = j0 + lane;
      const bool valid = j <= pos;
      bool ok = false;
      size_t row = 0, vat = 0;
      if (valid) {
        const int page = bt[j / ps];
        ok = (unsigned)page < (unsigned)num_pages;
        if (ok) {
          row = ((size_t)page * nkv + g) * ps + (j % ps);
          vat = ((size_t)page * nkv + g) * dv * ps + (j % ps);
        }
      }
      wpa_round<T>(qs, k_pages, v_pages, valid, ok, row, vat, (size_t)ps, (pos - j0 + 1) < 64 ? (pos - j0 + 1) : 64, d, dv,
                   scale, m, l, acc, ps_, rs_);
    }
  }
  if (sinks) {
    const float sk = sinks[h];
    const float m_new = fmaxf(m, sk);
    const float corr = expf(m - m_new);
    l = l * corr + expf(sk - m_new);
#pragma unroll
    for (int c = 0; c < WPA_MAX_D / 64; ++c) acc[c] *= corr;
  }
  T* o = out + (size_t)n * out_stride + (size_t)h * dv;
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int c = 0; c < WPA_MAX_D / 64; ++c) {
    const int dim = lane + 64 * c;
    if (dim < dv) o[dim] = from_float<T>(acc[c] * inv_l);
  }
}

extern "C" int ia_wpa_attention(const void* q, int q_stride, const void* k_pages, const void* v_pages,
                                const void* pk_pages, const void* pv_pages, void* out, int out_stride, int dtype,
                                const float* sinks, const int* token_seq, const int* positions, const int* bt_tok,
                                int bt_tok_stride, const int* bt_pool, int bt_pool_stride, int N, int nh, int nkv, int d,
                                int dv, int ps, int num_pages, int num_pool_pages, float scale, int window, int P,
                                hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || d <= 0 || dv <= 0 || d > WPA_MAX_D || dv > WPA_MAX_D || ps <= 0 ||
      num_pages <= 0 || bt_tok_stride <= 0 || window < 0 || P < 0 || q_stride < nh * d || out_stride < nh * dv)
    return IA_ERR_BAD_ARG;
  if (P > 0 && window > 0 && (!pk_pages || !pv_pages || !bt_pool || bt_pool_stride <= 0 || num_pool_pages <= 0))
    return IA_ERR_BAD_ARG;
  if (nh > 65535) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  if (!q || !k_pages || !v_pages || !out || !token_seq || !positions || !bt_tok) return IA_ERR_BAD_ARG;
  dim3 grid(N, nh);
  if (dtype == IA_F32)
    wpa_attention_kernel<float><<<grid, 64, 0, stream>>>(
        (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages, (const float*)pk_pages,
        (const float*)pv_pages, (float*)out, out_stride, sinks, token_seq, positions, bt_tok, bt_tok_stride, bt_pool,
        bt_pool_stride, nh, nkv, d, dv, ps, num_pages, num_pool_pages, scale, window, P);
  else if (dtype == IA_BF16)
    wpa_attention_kernel<bf16_t><<<grid, 64, 0, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (const bf16_t*)pk_pages,
        (const bf16_t*)pv_pages, (bf16_t*)out, out_stride, sinks, token_seq, positions, bt_tok, bt_tok_stride, bt_pool,
        bt_pool_stride, nh, nkv, d, dv, ps, num_pages, num_pool_pages, scale, window, P);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- rows divided by their root mean square, a wave a row
template <typename T>
__global__ __launch_bounds__(256) void rms_rows_kernel(const T* __restrict__ x, int x_stride, const void* __restrict__ w,
                                                       int w_dtype, T* __restrict__ y, int y_stride, int N, int C,
                                                       float eps) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (n >= N) return;
  const T* xr = x + (size_t)n * x_stride;
  float ss = 0.f;
  for (int i = lane; i < C; i += 64) {
    const float v = to_float(xr[i]);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)C + eps);
  T* yr = y + (size_t)n * y_stride;
  for (int i = lane; i < C; i += 64)
    yr[i] = from_float<T>(to_float(xr[i]) * inv * (w ? load_as_float(w, w_dtype, i) : 1.f));
}

extern "C" int ia_rms_rows(const void* x, int x_stride, const void* w, int w_dtype, void* y, int y_stride, int dtype,
                           int N, int C, float eps, hipStream_t stream) {
  if (N < 0 || C <= 0 || x_stride < C || y_stride < C || !(eps > 0.f)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!x || !y) return IA_ERR_BAD_ARG;
  const int grid = (N + 3) / 4;
  if (dtype == IA_F32)
    rms_rows_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, w, w_dtype, (float*)y, y_stride, N, C, eps);
  else if (dtype == IA_BF16)
    rms_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, w, w_dtype, (bf16_t*)y, y_stride, N, C,
                                                      eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- gelu_tanh(u) times a slice of a table's row of the token
__device__ __forceinline__ float wpa_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_mul_rows_kernel(const T* __restrict__ u, T* __restrict__ y,
                                                            const void* __restrict__ table, int t_dtype, int t_stride,
                                                            int col0, const int* __restrict__ ids, int vocab, long total,
                                                            int C) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const long n = i / C;
  const int j = (int)(i - n * C);
  const int id = ids[n];
  const float e = (unsigned)id < (unsigned)vocab ? load_as_float(table, t_dtype, (size_t)id * t_stride + col0 + j)
                                                 : __uint_as_float(0x7fc00000u);
  y[i] = from_float<T>(wpa_gelu_tanh(to_float(u[i])) * e);
}

extern "C" int ia_gelu_mul_rows(const void* u, void* y, int dtype, const void* table, int t_dtype, int t_stride,
                                int col0, const int* ids, int vocab, int N, int C, hipStream_t stream) {
  if (N < 0 || C <= 0 || col0 < 0 || t_stride < col0 + C || vocab <= 0) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!u || !y || !table || !ids) return IA_ERR_BAD_ARG;
  const long total = (long)N * C;
  const int grid = (int)((total + 255) / 256);
  if (dtype == IA_F32)
    gelu_mul_rows_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, (float*)y, table, t_dtype, t_stride, col0,
                                                          ids, vocab, total, C);
  else if (dtype == IA_BF16)
    gelu_mul_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, (bf16_t*)y, table, t_dtype, t_stride, col0,
                                                           ids, vocab, total, C);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_wpa_prepare)
IA_OP(ia_wpa_pool)
IA_OP(ia_wpa_attention)
IA_OP(ia_rms_rows)
IA_OP(ia_gelu_mul_rows)
