// Kernels for mixers that carry a little state from token to token beside (or in place of) the paged cache:
//
//   ia_causal_conv         a short causal convolution over time on every channel, the last taps-1 inputs of every
//                          request kept in its state slot (fp32), an optional bias on the input (a projection's),
//                          an optional bias on the output and an optional silu
//   ia_conv_state_update   the state of that convolution after a step
//   ia_causal_conv_single  both at once for steps in which every request brings one token
//   ia_qk_prepare          query and key heads between projection and attention: an RMS norm per head (one weight
//                          for all heads), rotation of neighbouring or half-split pairs with a factor on sine and
//                          cosine, the keys to their pages, and as values either the value heads of the row or the
//                          key heads as they came in
//   ia_ssd_scan            the selective state-space recurrence  S <- a S + dt B x^T,  y = S^T C + D x  per head,
//                          the state [N, P] of every request in its slot (fp32), token after token
//   ia_ssd_chunked         the same recurrence as matrix products over chunks of 64 tokens, for portions of prompts
//   ia_gated_group_norm    y * silu(z), then an RMS norm in equal parts of the row, times a weight
//   ia_concat_cast         rows [cast(a) | b]: the operand of a product over two streams side by side
//   ia_stream_add         the fp32 stream += a tensor or the partial sums of a split product
//   ia_stream_add2        the same for two of them one after the other, leaving the rounded stream as well
//   ia_add_bias, ia_softcap
//
// Everything between the loads and the stores is fp32: sums of squares, angles, decays, step sizes, the state.
// A row's result depends on its request's earlier tokens alone, in a fixed order of additions, so it is the same
// bits however a prompt is cut into steps and whatever else is in the batch.
#include "common.h"

// ------------------------------------------------------------------------------------------ convolution
// w [C, taps], or [taps, C] with tap_major.  u [N, >= C] (stride u_stride), state [slots, taps-1, C] fp32: state[slot][j] is the input at position
// ctx - (taps-1) + j of the request (zero before its start: a slot is cleared when it is taken).
// y[t] = b_out + sum_j w[c, j] (u[t - (taps-1) + j] + b_in), j ascending.
template <typename TU, typename TY>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const TU* __restrict__ u, int u_stride, const float* __restrict__ bias_in, const float* __restrict__ w,
    const float* __restrict__ bias_out, int act, TY* __restrict__ y, int y_stride, const float* __restrict__ state,
    long state_stride, const int* __restrict__ token_seq, const int* __restrict__ seq_starts,
    const int* __restrict__ state_slots, int N, int C, int taps, int tap_major) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (r >= N || c >= C) return;
  const int s = token_seq[r];
  const int i = r - seq_starts[s];
  const float* st = state + (size_t)state_slots[s] * state_stride;
  const float b_in = bias_in ? bias_in[c] : 0.f;
  float acc = bias_out ? bias_out[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int lag = taps - 1 - j;
    float v;
    if (i - lag >= 0)
      v = to_float(u[(size_t)(r - lag) * u_stride + c]) + b_in;
    else
      v = st[(size_t)(i - lag + taps - 1) * C + c];
    acc = __builtin_fmaf(tap_major ? w[(size_t)j * C + c] : w[(size_t)c * taps + j], v, acc);
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  y[(size_t)r * y_stride + c] = from_float<TY>(acc);
}

// The same for bf16 rows whose channels come in whole 16-byte pieces and weights stored tap by tap ([taps, C]: the
// weights of neighbouring channels are neighbours): a thread takes 8 channels of a row, the additions in the order
// of causal_conv_kernel.
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(
    const bf16_t* __restrict__ u, int u_stride, const float* __restrict__ bias_in, const float* __restrict__ w,
    const float* __restrict__ bias_out, int act, bf16_t* __restrict__ y, int y_stride, const float* __restrict__ state,
    long state_stride, const int* __restrict__ token_seq, const int* __restrict__ seq_starts,
    const int* __restrict__ state_slots, int N, int C, int taps) {
  const int r = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (r >= N || c >= C) return;
  const int s = token_seq[r];
  const int i = r - seq_starts[s];
  const float* st = state + (size_t)state_slots[s] * state_stride;
  float b_in[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (bias_in) {
    const float4 lo = *(const float4*)(bias_in + c), hi = *(const float4*)(bias_in + c + 4);
    b_in[0] = lo.x, b_in[1] = lo.y, b_in[2] = lo.z, b_in[3] = lo.w, b_in[4] = hi.x, b_in[5] = hi.y, b_in[6] = hi.z, b_in[7] = hi.w;
  }
  if (bias_out) {
    const float4 lo = *(const float4*)(bias_out + c), hi = *(const float4*)(bias_out + c + 4);
    acc[0] = lo.x, acc[1] = lo.y, acc[2] = lo.z, acc[3] = lo.w, acc[4] = hi.x, acc[5] = hi.y, acc[6] = hi.z, acc[7] = hi.w;
  }
  for (int j = 0; j < taps; ++j) {
    const int lag = taps - 1 - j;
    float v[8];
    if (i - lag >= 0) {
      const uint4 p = *(const uint4*)(u + (size_t)(r - lag) * u_stride + c);
      const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[2 * e] = __uint_as_float(pw[e] << 16) + b_in[2 * e];
        v[2 * e + 1] = __uint_as_float(pw[e] & 0xffff0000u) + b_in[2 * e + 1];
      }
    } else {
      const float* sp = st + (size_t)(i - lag + taps - 1) * C + c;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = sp[e];
    }
    const float4 w0 = *(const float4*)(w + (size_t)j * C + c), w1 = *(const float4*)(w + (size_t)j * C + c + 4);
    const float wj[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wj[e], v[e], acc[e]);
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float a = acc[2 * e], b = acc[2 * e + 1];
    if (act == 1) {
      a = a / (1.f + expf(-a));
      b = b / (1.f + expf(-b));
    }
    o[e] = (uint32_t)float_to_bf16_bits(a) | ((uint32_t)float_to_bf16_bits(b) << 16);
  }
  *(uint4*)(y + (size_t)r * y_stride + c) = make_uint4(o[0], o[1], o[2], o[3]);
}

// The same again for steps of many rows and at most four taps: a thread takes 8 channels of CONV_ROWS consecutive
// rows, loads every input row once for all the rows that reach it, and the weights once.
#define CONV_ROWS 4
__global__ __launch_bounds__(256) void causal_conv_rows_kernel(
    const bf16_t* __restrict__ u, int u_stride, const float* __restrict__ bias_in, const float* __restrict__ w,
    const float* __restrict__ bias_out, int act, bf16_t* __restrict__ y, int y_stride, const float* __restrict__ state,
    long state_stride, const int* __restrict__ token_seq, const int* __restrict__ seq_starts,
    const int* __restrict__ state_slots, int N, int C, int taps) {
  const int r0 = blockIdx.y * CONV_ROWS;
  const int c = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (r0 >= N || c >= C) return;
  float b_in[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, b_out[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (bias_in) {
    const float4 lo = *(const float4*)(bias_in + c), hi = *(const float4*)(bias_in + c + 4);
    b_in[0] = lo.x, b_in[1] = lo.y, b_in[2] = lo.z, b_in[3] = lo.w, b_in[4] = hi.x, b_in[5] = hi.y, b_in[6] = hi.z, b_in[7] = hi.w;
  }
  if (bias_out) {
    const float4 lo = *(const float4*)(bias_out + c), hi = *(const float4*)(bias_out + c + 4);
    b_out[0] = lo.x, b_out[1] = lo.y, b_out[2] = lo.z, b_out[3] = lo.w, b_out[4] = hi.x, b_out[5] = hi.y, b_out[6] = hi.z, b_out[7] = hi.w;
  }
  // input rows r0 - 3 .. r0 + CONV_ROWS - 1 of the step (those that exist), with the input bias
  float in[CONV_ROWS + 3][8];
#pragma unroll
  for (int k = 0; k < CONV_ROWS + 3; ++k) {
    const int r = r0 - 3 + k;
    uint4 p = make_uint4(0, 0, 0, 0);
    if (r >= 0 && r < N) p = *(const uint4*)(u + (size_t)r * u_stride + c);
    const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      in[k][2 * e] = __uint_as_float(pw[e] << 16) + b_in[2 * e];
      in[k][2 * e + 1] = __uint_as_float(pw[e] & 0xffff0000u) + b_in[2 * e + 1];
    }
  }
  // the weights by how far back their tap reaches (lag 0: the row itself), so that every index is known to the compiler
  float wt[4][8];
#pragma unroll
  for (int lag = 0; lag < 4; ++lag) {
    float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w1 = w0;
    if (lag < taps) {
      w0 = *(const float4*)(w + (size_t)(taps - 1 - lag) * C + c);
      w1 = *(const float4*)(w + (size_t)(taps - 1 - lag) * C + c + 4);
    }
    wt[lag][0] = w0.x, wt[lag][1] = w0.y, wt[lag][2] = w0.z, wt[lag][3] = w0.w;
    wt[lag][4] = w1.x, wt[lag][5] = w1.y, wt[lag][6] = w1.z, wt[lag][7] = w1.w;
  }
#pragma unroll
  for (int k = 0; k < CONV_ROWS; ++k) {
    const int r = r0 + k;
    if (r < N) {
      const int s = token_seq[r];
      const int i = r - seq_starts[s];
      const float* st = state + (size_t)state_slots[s] * state_stride;
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = b_out[e];
#pragma unroll
      for (int lag = 3; lag >= 0; --lag) {               // taps in ascending order
        if (lag < taps) {
          float v[8];
          if (i - lag >= 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = in[k + 3 - lag][e];
          } else {
            const float* sp = st + (size_t)(i - lag + taps - 1) * C + c;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = sp[e];
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(wt[lag][e], v[e], acc[e]);
        }
      }
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = acc[2 * e], b = acc[2 * e + 1];
        if (act == 1) {
          a = a / (1.f + expf(-a));
          b = b / (1.f + expf(-b));
        }
        o[e] = (uint32_t)float_to_bf16_bits(a) | ((uint32_t)float_to_bf16_bits(b) << 16);
      }
      *(uint4*)(y + (size_t)r * y_stride + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

// After the step: state[slot][j] <- the input at position ctx + q - (taps-1) + j, from this step's rows or from the
// old state (read in ascending j before the places are written: a thread owns its channel's taps-1 values).
template <typename TU>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const TU* __restrict__ u, int u_stride, const float* __restrict__ bias_in, float* __restrict__ state,
    long state_stride, const int* __restrict__ seq_starts, const int* __restrict__ state_slots, int B, int C, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (s >= B || c >= C) return;
  const int first = seq_starts[s], q = seq_starts[s + 1] - first;
  float* st = state + (size_t)state_slots[s] * state_stride;
  const float b_in = bias_in ? bias_in[c] : 0.f;
  for (int j = 0; j < taps - 1; ++j) {
    const int i = q - (taps - 1) + j;          // row of the request in this step, negative: before it
    float v;
    if (i >= 0)
      v = to_float(u[(size_t)(first + i) * u_stride + c]) + b_in;
    else
      v = st[(size_t)(j + q) * C + c];
    st[(size_t)j * C + c] = v;
  }
}

// For steps in which every request brings one token: the convolution and the state's move in one pass.  A thread
// owns a channel of a request: it reads the taps-1 kept inputs, adds in the order of causal_conv_kernel, and writes
// them back one place down with the new input last.
template <typename TU, typename TY>
__global__ __launch_bounds__(256) void causal_conv_single_kernel(
    const TU* __restrict__ u, int u_stride, const float* __restrict__ bias_in, const float* __restrict__ w,
    const float* __restrict__ bias_out, int act, TY* __restrict__ y, int y_stride, float* __restrict__ state,
    long state_stride, const int* __restrict__ token_seq, const int* __restrict__ state_slots, int N, int C, int taps,
    int tap_major) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (r >= N || c >= C) return;
  float* st = state + (size_t)state_slots[token_seq[r]] * state_stride;
  float acc = bias_out ? bias_out[c] : 0.f;
  const float cur = to_float(u[(size_t)r * u_stride + c]) + (bias_in ? bias_in[c] : 0.f);
  for (int j = 0; j < taps - 1; ++j) {
    const float v = st[(size_t)j * C + c];
    acc = __builtin_fmaf(tap_major ? w[(size_t)j * C + c] : w[(size_t)c * taps + j], v, acc);
    if (j > 0) st[(size_t)(j - 1) * C + c] = v;
  }
  acc = __builtin_fmaf(tap_major ? w[(size_t)(taps - 1) * C + c] : w[(size_t)c * taps + taps - 1], cur, acc);
  if (taps > 1) st[(size_t)(taps - 2) * C + c] = cur;
  if (act == 1) acc = acc / (1.f + expf(-acc));
  y[(size_t)r * y_stride + c] = from_float<TY>(acc);
}

// Every request of the step brings exactly one token (row r is request token_seq[r]'s): what ia_causal_conv and
// ia_conv_state_update do one after the other, the same bits.
extern "C" int ia_causal_conv_single(const void* u, int u_code, int u_stride, const float* bias_in, const float* w,
                                     const float* bias_out, int act, void* y, int y_code, int y_stride, float* state,
                                     long state_stride, const int* token_seq, const int* state_slots, int N, int C, int taps,
                                     int tap_major, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!u || !w || !y || !state || !token_seq || !state_slots || C <= 0 || taps < 1 || u_stride < C || y_stride < C ||
      N < 0 || N > 65535 || state_stride < (long)(taps - 1) * C || (act != 0 && act != 1))
    return IA_ERR_BAD_ARG;
  const dim3 grid((unsigned)((C + 255) / 256), (unsigned)N);
#define IA_CONV1(TU, TY)                                                                                               \
  causal_conv_single_kernel<TU, TY><<<grid, 256, 0, stream>>>((const TU*)u, u_stride, bias_in, w, bias_out, act, (TY*)y, \
                                                              y_stride, state, state_stride, token_seq, state_slots, N, C, taps, tap_major)
  if (u_code == IA_F32 && y_code == IA_F32) IA_CONV1(float, float);
  else if (u_code == IA_BF16 && y_code == IA_BF16) IA_CONV1(bf16_t, bf16_t);
  else if (u_code == IA_F32 && y_code == IA_BF16) IA_CONV1(float, bf16_t);
  else if (u_code == IA_BF16 && y_code == IA_F32) IA_CONV1(bf16_t, float);
  else return IA_ERR_BAD_ARG;
#undef IA_CONV1
  IA_LAUNCH_CHECK();
  return IA_OK;
}

extern "C" int ia_causal_conv(const void* u, int u_code, int u_stride, const float* bias_in, const float* w,
                              const float* bias_out, int act, void* y, int y_code, int y_stride, const float* state,
                              long state_stride, const int* token_seq, const int* seq_starts, const int* state_slots, int N, int C,
                              int taps, int tap_major, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!u || !w || !y || !state || !token_seq || !seq_starts || !state_slots || C <= 0 || taps < 1 || u_stride < C ||
      y_stride < C || N < 0 || N > 65535 || state_stride < (long)(taps - 1) * C || (act != 0 && act != 1))
    return IA_ERR_BAD_ARG;
  if (tap_major && u_code == IA_BF16 && y_code == IA_BF16 && C % 8 == 0 && !((uintptr_t)w & 15) &&
      !((uintptr_t)bias_in & 15) && !((uintptr_t)bias_out & 15) && u_stride % 8 == 0 && y_stride % 8 == 0 &&
      !((uintptr_t)u & 15) && !((uintptr_t)y & 15)) {
    if (taps <= 4 && N >= 64) {
      const dim3 rgrid((unsigned)((C / 8 + 255) / 256), (unsigned)((N + CONV_ROWS - 1) / CONV_ROWS));
      causal_conv_rows_kernel<<<rgrid, 256, 0, stream>>>((const bf16_t*)u, u_stride, bias_in, w, bias_out, act, (bf16_t*)y,
                                                         y_stride, state, state_stride, token_seq, seq_starts, state_slots, N, C, taps);
      IA_LAUNCH_CHECK();
      return IA_OK;
    }
    const dim3 vgrid((unsigned)((C / 8 + 255) / 256), (unsigned)N);
    causal_conv_vec_kernel<<<vgrid, 256, 0, stream>>>((const bf16_t*)u, u_stride, bias_in, w, bias_out, act, (bf16_t*)y,
                                                      y_stride, state, state_stride, token_seq, seq_starts, state_slots, N, C, taps);
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
  const dim3 grid((unsigned)((C + 255) / 256), (unsigned)N);
#define IA_CONV(TU, TY)                                                                                          \
  causal_conv_kernel<TU, TY><<<grid, 256, 0, stream>>>((const TU*)u, u_stride, bias_in, w, bias_out, act, (TY*)y, \
                                                       y_stride, state, state_stride, token_seq, seq_starts, state_slots, N, C, taps, tap_major)
  if (u_code == IA_F32 && y_code == IA_F32) IA_CONV(float, float);
  else if (u_code == IA_BF16 && y_code == IA_BF16) IA_CONV(bf16_t, bf16_t);
  else if (u_code == IA_F32 && y_code == IA_BF16) IA_CONV(float, bf16_t);
  else if (u_code == IA_BF16 && y_code == IA_F32) IA_CONV(bf16_t, float);
  else return IA_ERR_BAD_ARG;
#undef IA_CONV
  IA_LAUNCH_CHECK();
  return IA_OK;
}

extern "C" int ia_conv_state_update(const void* u, int u_code, int u_stride, const float* bias_in, float* state,
                                    long state_stride, const int* seq_starts, const int* state_slots, int B, int C, int taps,
                                    hipStream_t stream) {
  if (B == 0 || taps <= 1) return IA_OK;
  if (!u || !state || !seq_starts || !state_slots || C <= 0 || u_stride < C || B < 0 || B > 65535 ||
      state_stride < (long)(taps - 1) * C)
    return IA_ERR_BAD_ARG;
  const dim3 grid((unsigned)((C + 255) / 256), (unsigned)B);
  if (u_code == IA_F32)
    conv_state_update_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, u_stride, bias_in, state, state_stride,
                                                             seq_starts, state_slots, B, C, taps);
  else if (u_code == IA_BF16)
    conv_state_update_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, u_stride, bias_in, state, state_stride,
                                                              seq_starts, state_slots, B, C, taps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------------------------------ queries and keys
// One wave per (token, head).  Rows of x: nh query heads, nkv key heads, and nkv value heads when the values are
// not the keys.  pairing 0: value i with value i + rot/2; 1: value 2i with value 2i+1.
template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(
    const T* __restrict__ x, int x_stride, T* __restrict__ q_out, int q_stride, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float eps, const int* __restrict__ positions, const int* __restrict__ slots,
    const void* __restrict__ freq, int freq_f64, int rot, int pairing, float magnitude, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int N, int nh, int nkv, int d, int page_size, int num_pages, int values_are_keys) {
  const int lane = threadIdx.x & 63;
  const int heads = nh + nkv;
  const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long)N * heads) return;
  const int t = (int)(item / heads), hd = (int)(item % heads);
  const bool is_key = hd >= nh;
  if (is_key && !k_pages) return;
  const T* src = x + (size_t)t * x_stride + (size_t)hd * d;
  const float* wn = is_key ? k_norm : q_norm;
  // the norm: sum of squares over the head, lanes strided, joined across the wave in a fixed order
  float ss = 0.f;
  for (int i = lane; i < d; i += 64) {
    const float v = to_float(src[i]);
    ss = __builtin_fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = wn ? 1.0f / sqrtf(ss / (float)d + eps) : 1.0f;
  const int pos = positions[t];
  T* dst;
  if (is_key) {
    const int slot = slots[t];
    const int page = slot / page_size, off = slot - page * page_size;
    if (page < 0 || page >= num_pages) return;
    const int g = hd - nh;
    dst = k_pages + (((size_t)page * nkv + g) * page_size + off) * d;
    // the values: the value head of the row, or the key head as it came in; transposed within the page
    const T* vsrc = values_are_keys ? src : x + (size_t)t * x_stride + (size_t)(heads + g) * d;
    T* vdst = v_pages + ((size_t)page * nkv + g) * (size_t)d * page_size + off;
    for (int i = lane; i < d; i += 64) vdst[(size_t)i * page_size] = vsrc[i];
  } else {
    dst = q_out + (size_t)t * q_stride + (size_t)hd * d;
  }
  const int half = rot >> 1;
  // rotated pairs first, then the values that pass
  for (int p = lane; p < half; p += 64) {
    const int ia = pairing ? 2 * p : p, ib = pairing ? 2 * p + 1 : p + half;
    float a = to_float(src[ia]) * inv, b = to_float(src[ib]) * inv;
    if (wn) { a *= wn[ia]; b *= wn[ib]; }
    float sn, cs, lo, hi;
    rope_sincos(pos, freq, freq_f64, p, sn, cs);
    sn *= magnitude;
    cs *= magnitude;
    rope_pair(a, b, cs, sn, lo, hi);
    dst[ia] = from_float<T>(lo);
    dst[ib] = from_float<T>(hi);
  }
  for (int i = rot + lane; i < d; i += 64) {
    float a = to_float(src[i]) * inv;
    if (wn) a *= wn[i];
    dst[i] = from_float<T>(a);
  }
}

// The same for bf16 heads of whole 16-byte pieces whose rotated pairs are neighbours (or that are not rotated):
// a group of GL lanes (a power of two, at least d / 8) per (token, head), a lane takes 8 consecutive values, so a
// pair lies within a lane and every access but the transposed values' is 16 bytes.
__global__ __launch_bounds__(256) void qk_prepare_vec_kernel(
    const bf16_t* __restrict__ x, int x_stride, bf16_t* __restrict__ q_out, int q_stride, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float eps, const int* __restrict__ positions, const int* __restrict__ slots,
    const void* __restrict__ freq, int freq_f64, int rot, float magnitude, bf16_t* __restrict__ k_pages,
    bf16_t* __restrict__ v_pages, int N, int nh, int nkv, int d, int page_size, int num_pages, int values_are_keys, int GL) {
  const int heads = nh + nkv;
  const int per_block = 256 / GL;
  const long item = (long)blockIdx.x * per_block + threadIdx.x / GL;
  const int ch = threadIdx.x % GL;                        // which 8 values of the head
  const bool in_range = item < (long)N * heads;           // lanes past the end go along for the shuffles, idle
  const int t = in_range ? (int)(item / heads) : 0, hd = in_range ? (int)(item % heads) : 0;
  const bool live = in_range && 8 * ch < d;
  const bool is_key = hd >= nh;
  const bf16_t* src = x + (size_t)t * x_stride + (size_t)hd * d + 8 * ch;
  const float* wn = is_key ? k_norm : q_norm;
  uint4 raw = make_uint4(0, 0, 0, 0);
  if (live) raw = *(const uint4*)src;
  const uint32_t rw[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[2 * e] = __uint_as_float(rw[e] << 16);
    v[2 * e + 1] = __uint_as_float(rw[e] & 0xffff0000u);
  }
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(v[e], v[e], ss);
  for (int o = GL >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, IA_WAVE);
  if (!live || (is_key && !k_pages)) return;
  const int slot = is_key ? slots[t] : 0;
  const int page = slot / page_size, off = slot - page * page_size;
  if (is_key && (page < 0 || page >= num_pages)) return;
  const int g = hd - nh;
  if (is_key) {
    // the values: the value head of the row, or the key head as it came in; transposed within the page
    uint4 vr = raw;
    if (!values_are_keys) vr = *(const uint4*)(x + (size_t)t * x_stride + (size_t)(heads + g) * d + 8 * ch);
    const uint32_t vw[4] = {vr.x, vr.y, vr.z, vr.w};
    uint16_t* vdst = (uint16_t*)v_pages + ((size_t)page * nkv + g) * (size_t)d * page_size + (size_t)(8 * ch) * page_size + off;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      vdst[(size_t)(2 * e) * page_size] = (uint16_t)(vw[e] & 0xffffu);
      vdst[(size_t)(2 * e + 1) * page_size] = (uint16_t)(vw[e] >> 16);
    }
  }
  if (wn) {
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    const float4 w0 = *(const float4*)(wn + 8 * ch), w1 = *(const float4*)(wn + 8 * ch + 4);
    const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = v[e] * inv * wv[e];
  }
  const int pos = positions[t];
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    if (8 * ch + e < rot) {
      float sn, cs, lo, hi;
      rope_sincos(pos, freq, freq_f64, (8 * ch + e) >> 1, sn, cs);
      sn *= magnitude;
      cs *= magnitude;
      rope_pair(v[e], v[e + 1], cs, sn, lo, hi);
      v[e] = lo;
      v[e + 1] = hi;
    }
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = (uint32_t)float_to_bf16_bits(v[2 * e]) | ((uint32_t)float_to_bf16_bits(v[2 * e + 1]) << 16);
  bf16_t* dst = is_key ? k_pages + (((size_t)page * nkv + g) * page_size + off) * d + 8 * ch
                       : q_out + (size_t)t * q_stride + (size_t)hd * d + 8 * ch;
  *(uint4*)dst = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int ia_qk_prepare(const void* x, int code, int x_stride, void* q_out, int q_stride, const float* q_norm,
                             const float* k_norm, float eps, const int* positions, const int* slots, const void* freq,
                             int freq_f64, int rot, int pairing, float magnitude, void* k_pages, void* v_pages, int N,
                             int nh, int nkv, int d, int page_size, int num_pages, int values_are_keys,
                             hipStream_t stream) {
  if (N == 0) return IA_OK;
  const int write = k_pages != nullptr;
  if (!x || !q_out || !positions || N < 0 || nh <= 0 || nkv < 0 || d <= 0 || rot < 0 || rot > d || (rot & 1) ||
      (rot > 0 && !freq) || (write && (!v_pages || !slots || page_size <= 0 || num_pages <= 0)) ||
      x_stride < (nh + (write ? (values_are_keys ? nkv : 2 * nkv) : 0)) * d || q_stride < nh * d ||
      (q_norm == nullptr) != (k_norm == nullptr))
    return IA_ERR_BAD_ARG;
  // the rotation reads its pair from the source and writes both places: in place only where source and
  // destination are the same element for element (q_out == x with equal strides), which this launch allows
  const long items = (long)N * (nh + nkv);
  if (code == IA_BF16 && (pairing == 1 || rot == 0) && d % 8 == 0 && d <= 512 && x_stride % 8 == 0 && q_stride % 8 == 0 &&
      !((uintptr_t)x & 15) && !((uintptr_t)q_out & 15) && !((uintptr_t)k_pages & 15) && !((uintptr_t)q_norm & 15) &&
      !((uintptr_t)k_norm & 15)) {
    int GL = 1;
    while (8 * GL < d) GL <<= 1;
    const int per_block = 256 / GL;
    qk_prepare_vec_kernel<<<(unsigned)((items + per_block - 1) / per_block), 256, 0, stream>>>(
        (const bf16_t*)x, x_stride, (bf16_t*)q_out, q_stride, q_norm, k_norm, eps, positions, slots, freq, freq_f64, rot,
        magnitude, (bf16_t*)k_pages, (bf16_t*)v_pages, N, nh, nkv, d, page_size, num_pages, values_are_keys, GL);
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
  const unsigned grid = (unsigned)((items + 3) / 4);
  if (code == IA_F32)
    qk_prepare_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, (float*)q_out, q_stride, q_norm, k_norm,
                                                      eps, positions, slots, freq, freq_f64, rot, pairing, magnitude,
                                                      (float*)k_pages, (float*)v_pages, N, nh, nkv, d, page_size,
                                                      num_pages, values_are_keys);
  else if (code == IA_BF16)
    qk_prepare_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, (bf16_t*)q_out, q_stride, q_norm,
                                                       k_norm, eps, positions, slots, freq, freq_f64, rot, pairing,
                                                       magnitude, (bf16_t*)k_pages, (bf16_t*)v_pages, N, nh, nkv, d,
                                                       page_size, num_pages, values_are_keys);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------------------------------ the recurrence
// One workgroup per (request, head).  Thread (part, p) keeps the state values S[n][p] for n = part, part + parts,
// ... in registers over the request's tokens of this step; per token the parts' shares of y[p] = sum_n S[n][p] C[n]
// meet in LDS and are added in the order of the parts.  xbc rows: [x: nh P | B: G N | C: G N] after their
// convolution; dt rows: nh raw step sizes.  y [T, nh P] fp32.
template <typename T, int KMAX>
__global__ __launch_bounds__(256) void ssd_scan_kernel(
    const T* __restrict__ xbc, int xbc_stride, const T* __restrict__ dt_raw, int dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
    float* __restrict__ state, long state_stride, float* __restrict__ y, const int* __restrict__ seq_starts,
    const int* __restrict__ state_slots, int nh, int P, int Ns, int G, int parts) {
  extern __shared__ float lds[];
  float* bc = lds;                       // [2][2 Ns]: B and C of a token, two tokens in turn
  float* ysum = lds + 4 * Ns;            // [parts][P]
  const int s = blockIdx.y, hd = blockIdx.x;
  const int first = seq_starts[s], q = seq_starts[s + 1] - first;
  const int g = hd / (nh / G);
  const int tid = threadIdx.x;
  const int p = tid % P, part = tid / P;
  const bool live = part < parts;
  float* S = state + (size_t)state_slots[s] * state_stride + (size_t)hd * Ns * P;
  float reg[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; ++k) {
    const int n = part + k * parts;
    reg[k] = (live && n < Ns) ? S[(size_t)n * P + p] : 0.f;
  }
  const float A = -expf(a_log[hd]);
  const float bias = dt_bias[hd], D = skip[hd];
  const size_t b_col = (size_t)nh * P + (size_t)g * Ns, c_col = (size_t)nh * P + (size_t)G * Ns + (size_t)g * Ns;
  for (int i = 0; i < q; ++i) {
    const size_t row = (size_t)(first + i);
    float* cur = bc + (i & 1) * 2 * Ns;
    for (int n = tid; n < 2 * Ns; n += blockDim.x)
      cur[n] = to_float(xbc[row * xbc_stride + (n < Ns ? b_col + n : c_col + (n - Ns))]);
    const float z = to_float(dt_raw[row * dt_stride + hd]) + bias;
    const float dt = z > 20.f ? z : log1pf(expf(z));
    const float decay = expf(A * dt);
    const float xv = live ? to_float(xbc[row * xbc_stride + (size_t)hd * P + p]) : 0.f;
    const float dx = dt * xv;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int n = part + k * parts;
      if (n < Ns) {
        reg[k] = __builtin_fmaf(decay, reg[k], dx * cur[n]);
        acc = __builtin_fmaf(reg[k], cur[Ns + n], acc);
      }
    }
    if (live) ysum[part * P + p] = acc;
    __syncthreads();
    if (part == 0) {
      float t = ysum[p];
      for (int k = 1; k < parts; ++k) t += ysum[k * P + p];
      y[row * ((size_t)nh * P) + (size_t)hd * P + p] = __builtin_fmaf(D, xv, t);
    }
    // the next token's B and C go to the other half of bc; ysum is read before the next token's barrier pair ends
  }
  if (live) {
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      const int n = part + k * parts;
      if (n < Ns) S[(size_t)n * P + p] = reg[k];
    }
  }
}

extern "C" int ia_ssd_scan(const void* xbc, int code, int xbc_stride, const void* dt_raw, int dt_stride,
                           const float* dt_bias, const float* a_log, const float* skip, float* state, long state_stride,
                           float* y, const int* seq_starts, const int* state_slots, int B, int nh, int P, int Ns, int G,
                           hipStream_t stream) {
  if (B == 0) return IA_OK;
  if (!xbc || !dt_raw || !dt_bias || !a_log || !skip || !state || !y || !seq_starts || !state_slots || B < 0 ||
      B > 65535 || nh <= 0 || P <= 0 || P > 256 || Ns <= 0 || G <= 0 || nh % G || xbc_stride < nh * P + 2 * G * Ns ||
      dt_stride < nh || state_stride < (long)nh * Ns * P)
    return IA_ERR_BAD_ARG;
  int parts = 256 / P;
  if (parts > Ns) parts = Ns;
  const int per = (Ns + parts - 1) / parts;
  if (per > 128) return IA_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)nh, (unsigned)B);
  const size_t lds = sizeof(float) * (4 * (size_t)Ns + (size_t)parts * P);
  if (lds > 64 * 1024) return IA_ERR_UNSUPPORTED;
#define IA_SCAN(T, KM)                                                                                            \
  ssd_scan_kernel<T, KM><<<grid, 256, lds, stream>>>((const T*)xbc, xbc_stride, (const T*)dt_raw, dt_stride, dt_bias, \
                                                     a_log, skip, state, state_stride, y, seq_starts, state_slots, nh, P, Ns, G,  \
                                                     parts)
#define IA_SCAN_K(T)                       \
  do {                                     \
    if (per <= 8) IA_SCAN(T, 8);           \
    else if (per <= 16) IA_SCAN(T, 16);    \
    else if (per <= 32) IA_SCAN(T, 32);    \
    else if (per <= 64) IA_SCAN(T, 64);    \
    else IA_SCAN(T, 128);                  \
  } while (0)
  if (code == IA_F32) IA_SCAN_K(float);
  else if (code == IA_BF16) IA_SCAN_K(bf16_t);
  else return IA_ERR_BAD_ARG;
#undef IA_SCAN_K
#undef IA_SCAN
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------------------------------ the recurrence, in chunks
// The same recurrence for steps that bring portions of prompts, as matrix products over chunks of 64 tokens.  With
// a_i = -exp(a_log) dt_i and c_i = a_1 + ... + a_i inside a chunk that starts from the state S0:
//
//   y_i = exp(c_i) C_i^T S0 + sum_{j <= i} exp(c_i - c_j) dt_j (C_i . B_j) x_j + D x_i
//   S   = exp(c_L) S0 + sum_j exp(c_L - c_j) dt_j B_j x_j^T
//
// One workgroup of four waves per (request, head, 16 of the head's P values) walks the request's chunks in order.
// C B^T is a bf16 product (B and C are bf16 values as stored, so nothing is rounded) with fp32 sums; everything that
// carries a decay, a step size or the state is fp32 on v_mfma_f32_16x16x4_f32: every exponent is at most zero.  The
// state of the slice lives in LDS between chunks.  Rows past a request's last token are zero with dt = 0, which
// leaves sums and state as they are.
typedef __bf16 sm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sm_f32x4 __attribute__((ext_vector_type(4)));

#define SSD_L 64          // tokens of a chunk
#define SSD_PW 16         // values of a head that a workgroup owns
#define SSD_GS 68         // row stride of the chunk's [L, L] matrix in LDS, floats
#define SSD_XS 20         // row stride of x and of the state in LDS, floats

// What a thread holds of the next chunk while the current one is computed.
#define SSD_MAXV 4        // 16-byte pieces of B (and of C) a thread loads per chunk: 64 rows of up to 128 values

__global__ __launch_bounds__(256) void ssd_chunk_kernel(
    const bf16_t* __restrict__ xbc, int xbc_stride, const bf16_t* __restrict__ dt_raw, int dt_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ skip,
    float* __restrict__ state, long state_stride, float* __restrict__ y, const int* __restrict__ seq_starts,
    const int* __restrict__ state_slots, int nh, int P, int Ns, int G, int NP) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssd_lds[];
  const int BS = NP + 8;                                   // row stride of B and C in LDS, bf16 values
  uint16_t* Bs = (uint16_t*)ssd_lds;                       // [L][BS]
  uint16_t* Cs = Bs + SSD_L * BS;                          // [L][BS]
  float* Gs = (float*)(Cs + SSD_L * BS);                   // [L][GS]
  float* Xs = Gs + SSD_L * SSD_GS;                         // [L][XS]
  float* Ss = Xs + SSD_L * SSD_XS;                         // [Ns][XS]
  float* cum = Ss + (size_t)Ns * SSD_XS;                   // [L] running sum of a
  float* dts = cum + SSD_L;                                // [L] step sizes
  float* ecs = dts + SSD_L;                                // [L] exp(c_i)
  float* wts = ecs + SSD_L;                                // [L] exp(c_L - c_j) dt_j
  const int slices = P / SSD_PW;
  const int hd = blockIdx.x / slices, ps = blockIdx.x - hd * slices;
  const int s = blockIdx.y;
  const int first = seq_starts[s], q = seq_starts[s + 1] - first;
  if (q <= 0) return;
  const int g = hd / (nh / G);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l15 = lane & 15, kk = lane >> 4;
  float* S = state + (size_t)state_slots[s] * state_stride + (size_t)hd * Ns * P + (size_t)ps * SSD_PW;
  const float A = -expf(a_log[hd]);
  const float bias = dt_bias[hd], D = skip[hd];
  const size_t x_col = (size_t)hd * P + (size_t)ps * SSD_PW;
  const size_t b_col = (size_t)nh * P + (size_t)g * Ns, c_col = b_col + (size_t)G * Ns;
  const int yw = nh * P;
  // the state of the slice, and zeros in the columns of B and C past the state's size
  for (int i = tid; i < Ns * SSD_PW; i += 256) Ss[(i >> 4) * SSD_XS + (i & 15)] = S[(size_t)(i >> 4) * P + (i & 15)];
  if (NP > Ns)
    for (int i = tid; i < SSD_L * (NP - Ns); i += 256) {
      const int r = i / (NP - Ns), c = Ns + i % (NP - Ns);
      Bs[r * BS + c] = 0;
      Cs[r * BS + c] = 0;
    }
  // a thread's pieces of a chunk: piece v of B and C is 8 values of row (tid + 256 v) / vec_row; x values 4 tid .. 4 tid + 3
  const int vec_row = Ns >> 3;                             // 16-byte pieces of a row of B or C (a power of two or not)
  int vr[SSD_MAXV], vc[SSD_MAXV];
#pragma unroll
  for (int v = 0; v < SSD_MAXV; ++v) {
    const int i = tid + 256 * v;
    vr[v] = i / vec_row;
    vc[v] = 8 * (i - vr[v] * vec_row);
    if (vr[v] >= SSD_L) vr[v] = -1;
  }
  const int xr = tid >> 2, xc = 4 * (tid & 3);
  uint4 nb_[SSD_MAXV], nc_[SSD_MAXV];
  uint2 nx_;
  float ndt;
  auto fetch = [&](int c0) {                               // the chunk's rows from memory into registers
    const int Lc = q - c0 < SSD_L ? q - c0 : SSD_L;
    const size_t row0 = (size_t)(first + c0);
#pragma unroll
    for (int v = 0; v < SSD_MAXV; ++v) {
      nb_[v] = make_uint4(0, 0, 0, 0);
      nc_[v] = nb_[v];
      if (vr[v] >= 0 && vr[v] < Lc) {
        const bf16_t* rp = xbc + (row0 + vr[v]) * xbc_stride;
        nb_[v] = *(const uint4*)(rp + b_col + vc[v]);
        nc_[v] = *(const uint4*)(rp + c_col + vc[v]);
      }
    }
    nx_ = make_uint2(0, 0);
    if (xr < Lc) nx_ = *(const uint2*)(xbc + (row0 + xr) * xbc_stride + x_col + xc);
    ndt = 0.f;
    if (wave == 0 && lane < Lc) ndt = to_float(dt_raw[(row0 + lane) * dt_stride + hd]);
  };
  fetch(0);
  for (int c0 = 0; c0 < q; c0 += SSD_L) {
    const int Lc = q - c0 < SSD_L ? q - c0 : SSD_L;
    const size_t row0 = (size_t)(first + c0);
    __syncthreads();                                       // the chunk before is done with B, C, x and the sums
    // ---- B, C, x of the chunk from the registers; step sizes, the running sum of a and what hangs on it
#pragma unroll
    for (int v = 0; v < SSD_MAXV; ++v)
      if (vr[v] >= 0) {
        *(uint4*)(Bs + vr[v] * BS + vc[v]) = nb_[v];
        *(uint4*)(Cs + vr[v] * BS + vc[v]) = nc_[v];
      }
    {
      float* xp = Xs + xr * SSD_XS + xc;
      xp[0] = __uint_as_float(nx_.x << 16);
      xp[1] = __uint_as_float(nx_.x & 0xffff0000u);
      xp[2] = __uint_as_float(nx_.y << 16);
      xp[3] = __uint_as_float(nx_.y & 0xffff0000u);
    }
    if (wave == 0) {
      float dt = 0.f;
      if (lane < Lc) {
        const float z = ndt + bias;
        dt = z > 20.f ? z : log1pf(expf(z));
      }
      float c = A * dt;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(c, o, 64);
        if (lane >= o) c += up;
      }
      const float clast = __shfl(c, 63, 64);
      cum[lane] = c;
      dts[lane] = dt;
      ecs[lane] = expf(c);
      wts[lane] = expf(clast - c) * dt;
    }
    if (c0 + SSD_L < q) fetch(c0 + SSD_L);                 // the next chunk is on its way while this one is computed
    __syncthreads();
    // ---- G[i][j] = (C_i . B_j) exp(c_i - c_j) dt_j for j <= i: the ten tiles of 16 x 16 on and under the diagonal,
    // wave w takes tiles w, w + 4, w + 8 of the list (0,0) (1,0) (1,1) (2,0) ... (3,3)
    for (int t = wave; t < 10; t += 4) {
      const int it = t < 1 ? 0 : t < 3 ? 1 : t < 6 ? 2 : 3;
      const int jt = t - (it * (it + 1) >> 1);
      sm_f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
      const uint16_t* cp = Cs + (16 * it + l15) * BS + 8 * kk;
      const uint16_t* bp = Bs + (16 * jt + l15) * BS + 8 * kk;
      for (int k0 = 0; k0 < NP; k0 += 64) {
        const sm_bf16x8 a0 = *(const sm_bf16x8*)(cp + k0), b0 = *(const sm_bf16x8*)(bp + k0);
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc0, 0, 0, 0);
        if (k0 + 32 < NP) {
          const sm_bf16x8 a1 = *(const sm_bf16x8*)(cp + k0 + 32), b1 = *(const sm_bf16x8*)(bp + k0 + 32);
          acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, acc1, 0, 0, 0);
        }
      }
      const int j = 16 * jt + l15;
      const float cj = cum[j], dj = dts[j];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * it + 4 * kk + r;
        Gs[i * SSD_GS + j] = j <= i ? (acc0[r] + acc1[r]) * expf(cum[i] - cj) * dj : 0.f;
      }
    }
    __syncthreads();
    // ---- y rows 16 w .. 16 w + 15 of the chunk: G x + exp(c_i) C S0 + D x, in three sums that run side by side
    {
      sm_f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc1 = acc, acc2 = acc;
      const int i = 16 * wave + l15;                       // the row this lane feeds
      for (int jb = 0; jb <= wave; ++jb) {
        const sm_f32x4 a = *(const sm_f32x4*)(Gs + i * SSD_GS + 16 * jb + 4 * kk);
        const float* xp = Xs + (16 * jb + 4 * kk) * SSD_XS + l15;
        const float x0 = xp[0], x1 = xp[SSD_XS], x2 = xp[2 * SSD_XS], x3 = xp[3 * SSD_XS];
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], x0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], x1, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], x2, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], x3, acc, 0, 0, 0);
      }
      const float ei = ecs[i];
      for (int nb = 0; nb < Ns; nb += 32) {
        const bool two = nb + 16 < Ns;
        const uint2 cw = *(const uint2*)(Cs + i * BS + nb + 4 * kk);
        const uint2 cv = two ? *(const uint2*)(Cs + i * BS + nb + 16 + 4 * kk) : make_uint2(0, 0);
        const float* sp = Ss + (nb + 4 * kk) * SSD_XS + l15;
        const float* sq = two ? sp + 16 * SSD_XS : sp;
        const float s0 = sp[0], s1 = sp[SSD_XS], s2 = sp[2 * SSD_XS], s3 = sp[3 * SSD_XS];
        const float t0 = sq[0], t1 = sq[SSD_XS], t2 = sq[2 * SSD_XS], t3 = sq[3 * SSD_XS];
        acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cw.x << 16) * ei, s0, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cv.x << 16) * ei, t0, acc2, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cw.x & 0xffff0000u) * ei, s1, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cv.x & 0xffff0000u) * ei, t1, acc2, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cw.y << 16) * ei, s2, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cv.y << 16) * ei, t2, acc2, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cw.y & 0xffff0000u) * ei, s3, acc1, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(cv.y & 0xffff0000u) * ei, t3, acc2, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int io = 16 * wave + 4 * kk + r;
        if (io < Lc)
          y[(row0 + io) * yw + x_col + l15] = __builtin_fmaf(D, Xs[io * SSD_XS + l15], acc[r] + (acc1[r] + acc2[r]));
      }
    }
    __syncthreads();                                       // every wave has read S0
    // ---- the state after the chunk: tiles of 16 state rows, wave w takes tiles w, w + 4, ..., two at a time
    {
      const float keep = ecs[SSD_L - 1];
      for (int nt = wave; 16 * nt < Ns; nt += 8) {
        const bool two = 16 * (nt + 4) < Ns;
        const int nu = two ? nt + 4 : nt;
        sm_f32x4 acc, acc1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          acc[r] = keep * Ss[(16 * nt + 4 * kk + r) * SSD_XS + l15];
          acc1[r] = keep * Ss[(16 * nu + 4 * kk + r) * SSD_XS + l15];
        }
#pragma unroll 2
        for (int jb = 0; jb < SSD_L; jb += 16) {
          const sm_f32x4 wj = *(const sm_f32x4*)(wts + jb + 4 * kk);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int j = jb + 4 * kk + r;
            const float xv = Xs[j * SSD_XS + l15];
            const float a = __uint_as_float((uint32_t)Bs[j * BS + 16 * nt + l15] << 16) * wj[r];
            const float a1 = __uint_as_float((uint32_t)Bs[j * BS + 16 * nu + l15] << 16) * wj[r];
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, xv, acc, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, xv, acc1, 0, 0, 0);
          }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          Ss[(16 * nt + 4 * kk + r) * SSD_XS + l15] = acc[r];
          if (two) Ss[(16 * nu + 4 * kk + r) * SSD_XS + l15] = acc1[r];
        }
      }
    }
  }
  __syncthreads();
  for (int i = tid; i < Ns * SSD_PW; i += 256) S[(size_t)(i >> 4) * P + (i & 15)] = Ss[(i >> 4) * SSD_XS + (i & 15)];
}

// Whether ia_ssd_chunked takes these sizes (otherwise ia_ssd_scan does the step).
extern "C" int ia_ssd_chunked_takes(int nh, int P, int Ns, int G, int xbc_stride) {
  return nh > 0 && G > 0 && nh % G == 0 && P % SSD_PW == 0 && Ns % 16 == 0 && Ns >= 16 && Ns <= 32 * SSD_MAXV && xbc_stride % 8 == 0;
}

extern "C" int ia_ssd_chunked(const void* xbc, int code, int xbc_stride, const void* dt_raw, int dt_stride,
                              const float* dt_bias, const float* a_log, const float* skip, float* state,
                              long state_stride, float* y, const int* seq_starts, const int* state_slots, int B, int nh,
                              int P, int Ns, int G, hipStream_t stream) {
  if (B == 0) return IA_OK;
  if (!xbc || !dt_raw || !dt_bias || !a_log || !skip || !state || !y || !seq_starts || !state_slots || B < 0 ||
      B > 65535 || nh <= 0 || P <= 0 || Ns <= 0 || G <= 0 || nh % G || xbc_stride < nh * P + 2 * G * Ns ||
      dt_stride < nh || state_stride < (long)nh * Ns * P || ((uintptr_t)xbc & 15))
    return IA_ERR_BAD_ARG;
  if (code != IA_BF16 || !ia_ssd_chunked_takes(nh, P, Ns, G, xbc_stride)) return IA_ERR_UNSUPPORTED;
  const int NP = (Ns + 31) / 32 * 32;
  const size_t lds = 2 * (size_t)SSD_L * (NP + 8) * 2 + sizeof(float) * ((size_t)SSD_L * SSD_GS + (size_t)SSD_L * SSD_XS +
                                                                        (size_t)Ns * SSD_XS + 4 * SSD_L);
  static size_t lds_allowed = 64 * 1024;
  if (lds > lds_allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)ssd_chunk_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(160 * 1024));
    if (e != hipSuccess) return (int)e;
    lds_allowed = 160 * 1024;
  }
  const dim3 grid((unsigned)(nh * (P / SSD_PW)), (unsigned)B);
  ssd_chunk_kernel<<<grid, 256, lds, stream>>>((const bf16_t*)xbc, xbc_stride, (const bf16_t*)dt_raw, dt_stride, dt_bias,
                                               a_log, skip, state, state_stride, y, seq_starts, state_slots, nh, P, Ns, G, NP);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------------------------------ gate and norm
// One workgroup per (row, part): out = unit_rms(y * silu(z)) * w over the part's `size` values.
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z,
                                                               int z_stride, const float* __restrict__ w,
                                                               T* __restrict__ out, int inner, int size, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.y, part = blockIdx.x;
  const size_t base = (size_t)part * size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < size; i += 256) {
    const float g = to_float(z[(size_t)r * z_stride + base + i]);
    const float v = y[(size_t)r * inner + base + i] * (g / (1.f + expf(-g)));
    ss = __builtin_fmaf(v, v, ss);
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)size + eps);
  for (int i = threadIdx.x; i < size; i += 256) {
    const float g = to_float(z[(size_t)r * z_stride + base + i]);
    const float v = y[(size_t)r * inner + base + i] * (g / (1.f + expf(-g)));
    out[(size_t)r * inner + base + i] = from_float<T>(v * inv * w[base + i]);
  }
}

// The same for parts of up to 256 PER values: a thread keeps its gated values between the sum and the store (one
// pass over y and z); the additions in the order of gated_group_norm_kernel.
template <typename T, int PER>
__global__ __launch_bounds__(256) void gated_group_norm_kept_kernel(const float* __restrict__ y, const T* __restrict__ z,
                                                                    int z_stride, const float* __restrict__ w,
                                                                    T* __restrict__ out, int inner, int size, float eps) {
  __shared__ float red[4];
  const int r = blockIdx.y, part = blockIdx.x;
  const size_t base = (size_t)part * size;
  float v[PER];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + 256 * k;
    v[k] = 0.f;
    if (i < size) {
      const float g = to_float(z[(size_t)r * z_stride + base + i]);
      v[k] = y[(size_t)r * inner + base + i] * (g / (1.f + expf(-g)));
      ss = __builtin_fmaf(v[k], v[k], ss);
    }
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)size + eps);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + 256 * k;
    if (i < size) out[(size_t)r * inner + base + i] = from_float<T>(v[k] * inv * w[base + i]);
  }
}

extern "C" int ia_gated_group_norm(const float* y, const void* z, int code, int z_stride, const float* w, void* out,
                                   int N, int inner, int groups, float eps, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!y || !z || !w || !out || N < 0 || N > 65535 || inner <= 0 || groups <= 0 || inner % groups || z_stride < inner)
    return IA_ERR_BAD_ARG;
  const dim3 grid((unsigned)groups, (unsigned)N);
  const int size = inner / groups;
  if (size <= 1024 && (code == IA_F32 || code == IA_BF16)) {
#define IA_GGN(T, PER)                                                                                                  \
  gated_group_norm_kept_kernel<T, PER><<<grid, 256, 0, stream>>>(y, (const T*)z, z_stride, w, (T*)out, inner, size, eps)
    if (code == IA_F32) { if (size <= 256) IA_GGN(float, 1); else if (size <= 512) IA_GGN(float, 2); else IA_GGN(float, 4); }
    else { if (size <= 256) IA_GGN(bf16_t, 1); else if (size <= 512) IA_GGN(bf16_t, 2); else IA_GGN(bf16_t, 4); }
#undef IA_GGN
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
  if (code == IA_F32)
    gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>(y, (const float*)z, z_stride, w, (float*)out, inner,
                                                            inner / groups, eps);
  else if (code == IA_BF16)
    gated_group_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, (const bf16_t*)z, z_stride, w, (bf16_t*)out, inner,
                                                             inner / groups, eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------------------------------ small row kernels
// out [N, 2 W] = [cast(a [N, W] fp32) | b [N, W]]
template <typename T>
__global__ __launch_bounds__(256) void concat_cast_kernel(const float* __restrict__ a, const T* __restrict__ b,
                                                          T* __restrict__ out, size_t n, int W) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const size_t r = i / W, c = i - r * W;
    out[r * 2 * W + c] = from_float<T>(a[i]);
    out[r * 2 * W + W + c] = b[i];
  }
}

extern "C" int ia_concat_cast(const float* a, const void* b, void* out, int code, int N, int W, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!a || !b || !out || N < 0 || W <= 0) return IA_ERR_BAD_ARG;
  const size_t n = (size_t)N * W;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (code == IA_F32) concat_cast_kernel<float><<<grid, 256, 0, stream>>>(a, (const float*)b, (float*)out, n, W);
  else if (code == IA_BF16) concat_cast_kernel<bf16_t><<<grid, 256, 0, stream>>>(a, (const bf16_t*)b, (bf16_t*)out, n, W);
  else return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// h [N, H] fp32 += delta, a tensor [N, H] or a stack of partial sums [splits, N, H], added in the order of their index
template <typename T>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ h, const T* __restrict__ delta, int splits,
                                                         size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) h[i] += load_split_sum(delta + i, splits, n);
}

extern "C" int ia_stream_add(float* h, const void* delta, int code, int splits, int N, int H, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!h || !delta || N < 0 || H <= 0 || splits < 1) return IA_ERR_BAD_ARG;
  const size_t n = (size_t)N * H;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (code == IA_F32) stream_add_kernel<float><<<grid, 256, 0, stream>>>(h, (const float*)delta, splits, n);
  else if (code == IA_BF16) stream_add_kernel<bf16_t><<<grid, 256, 0, stream>>>(h, (const bf16_t*)delta, splits, n);
  else return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// h += a, then h += b (nullable), each a tensor or a stack of partial sums as in ia_stream_add, the additions in that
// order; x (nullable) gets the new h in its own type: the two results of sublayers that ran side by side enter the
// stream in one pass, which also leaves the rounded stream for whoever reads it next.  Four values a thread.
__device__ __forceinline__ void sa2_load4(const void* p, int code, size_t i, float (&v)[4]) {
  if (code == IA_F32) {
    const float4 f = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
    v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
  } else {
    const uint2 u = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p) + i);
    v[0] = bf16_bits_to_float((uint16_t)(u.x & 0xffffu)); v[1] = bf16_bits_to_float((uint16_t)(u.x >> 16));
    v[2] = bf16_bits_to_float((uint16_t)(u.y & 0xffffu)); v[3] = bf16_bits_to_float((uint16_t)(u.y >> 16));
  }
}
__device__ __forceinline__ void sa2_sum4(const void* p, int code, int splits, size_t i, size_t n, float (&v)[4]) {
  sa2_load4(p, code, i, v);
  for (int k = 1; k < splits; ++k) {
    float w[4];
    sa2_load4(p, code, i + (size_t)k * n, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += w[e];
  }
}
template <bool VEC>
__global__ __launch_bounds__(256) void stream_add2_kernel(float* __restrict__ h, const void* __restrict__ a, int a_code,
                                                          int a_splits, const void* __restrict__ b, int b_code,
                                                          int b_splits, void* __restrict__ x, int x_code, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  if (VEC) {
    for (size_t i4 = (size_t)blockIdx.x * 256 + threadIdx.x; i4 < n / 4; i4 += stride) {
      const size_t i = i4 * 4;
      float hv[4], av[4];
      sa2_load4(h, IA_F32, i, hv);
      sa2_sum4(a, a_code, a_splits, i, n, av);
#pragma unroll
      for (int e = 0; e < 4; ++e) hv[e] += av[e];
      if (b) {
        sa2_sum4(b, b_code, b_splits, i, n, av);
#pragma unroll
        for (int e = 0; e < 4; ++e) hv[e] += av[e];
      }
      *reinterpret_cast<float4*>(h + i) = make_float4(hv[0], hv[1], hv[2], hv[3]);
      if (x) {
        if (x_code == IA_F32) {
          *reinterpret_cast<float4*>(reinterpret_cast<float*>(x) + i) = make_float4(hv[0], hv[1], hv[2], hv[3]);
        } else {
          uint2 u;
          u.x = (uint32_t)float_to_bf16_bits(hv[0]) | ((uint32_t)float_to_bf16_bits(hv[1]) << 16);
          u.y = (uint32_t)float_to_bf16_bits(hv[2]) | ((uint32_t)float_to_bf16_bits(hv[3]) << 16);
          *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(x) + i) = u;
        }
      }
    }
  } else {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
      float v = h[i];
      float t = load_as_float(a, a_code, i);
      for (int k = 1; k < a_splits; ++k) t += load_as_float(a, a_code, i + (size_t)k * n);
      v += t;
      if (b) {
        t = load_as_float(b, b_code, i);
        for (int k = 1; k < b_splits; ++k) t += load_as_float(b, b_code, i + (size_t)k * n);
        v += t;
      }
      h[i] = v;
      if (x) {
        if (x_code == IA_F32) reinterpret_cast<float*>(x)[i] = v;
        else reinterpret_cast<uint16_t*>(x)[i] = float_to_bf16_bits(v);
      }
    }
  }
}

extern "C" int ia_stream_add2(float* h, const void* a, int a_code, int a_splits, const void* b, int b_code, int b_splits,
                              void* x, int x_code, int N, int H, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!h || !a || N < 0 || H <= 0 || a_splits < 1 || (b && b_splits < 1)) return IA_ERR_BAD_ARG;
  if ((a_code != IA_F32 && a_code != IA_BF16) || (b && b_code != IA_F32 && b_code != IA_BF16) ||
      (x && x_code != IA_F32 && x_code != IA_BF16))
    return IA_ERR_BAD_ARG;
  const size_t n = (size_t)N * H;
  const auto aligned = [](const void* p, size_t to) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % to) == 0; };
  const bool vec = (n % 4) == 0 && aligned(h, 16) && aligned(a, 16) && aligned(b, 16) && aligned(x, 16);
  const size_t items = vec ? n / 4 : n;
  const unsigned grid = (unsigned)((items + 255) / 256 < 65536 ? (items + 255) / 256 : 65536);
  if (vec) stream_add2_kernel<true><<<grid, 256, 0, stream>>>(h, a, a_code, a_splits, b, b_code, b_splits, x, x_code, n);
  else stream_add2_kernel<false><<<grid, 256, 0, stream>>>(h, a, a_code, a_splits, b, b_code, b_splits, x, x_code, n);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// y [N, C] += bias (fp32 vector), rounded once
template <typename T>
__global__ __launch_bounds__(256) void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, size_t n, int C) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
    y[i] = from_float<T>(to_float(y[i]) + bias[i % C]);
}

extern "C" int ia_add_bias(void* y, int code, const float* bias, int N, int C, hipStream_t stream) {
  if (N == 0) return IA_OK;
  if (!y || !bias || N < 0 || C <= 0) return IA_ERR_BAD_ARG;
  const size_t n = (size_t)N * C;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (code == IA_F32) add_bias_kernel<float><<<grid, 256, 0, stream>>>((float*)y, bias, n, C);
  else if (code == IA_BF16) add_bias_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)y, bias, n, C);
  else return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// x <- cap * tanh(x / cap), fp32 in place
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, size_t n, float cap) {
  const size_t stride = (size_t)gridDim.x * 256;
  const float inv = 1.0f / cap;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) x[i] = cap * tanhf(x[i] * inv);
}

extern "C" int ia_softcap(float* x, int rows, int cols, float cap, hipStream_t stream) {
  if (rows == 0) return IA_OK;
  if (!x || rows < 0 || cols <= 0 || !(cap > 0.f)) return IA_ERR_BAD_ARG;
  const size_t n = (size_t)rows * cols;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  softcap_kernel<<<grid, 256, 0, stream>>>(x, n, cap);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_causal_conv)
IA_OP(ia_causal_conv_single)
IA_OP(ia_conv_state_update)
IA_OP(ia_qk_prepare)
IA_OP(ia_ssd_scan)
IA_OP(ia_ssd_chunked)
IA_OP(ia_gated_group_norm)
IA_OP(ia_concat_cast)
IA_OP(ia_stream_add)
IA_OP(ia_stream_add2)
IA_OP(ia_add_bias)
IA_OP(ia_softcap)
