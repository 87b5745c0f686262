// Gated linear attention: a recurrence per head over a state S [dim, vdim] of fp32 values with one decay per key
// channel and token,
//     S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,      o_t = S_t^T (c q_t),      alpha = sigmoid(z)^(1/tau),
// and what follows it: every head's o divided by its root mean square over vdim, times a weight shared by the heads,
// times silu(gate).
//
//   ia_gla_scan         the recurrence token after token for the rows of every request of a step, from the request's
//                       state slot, which it leaves moved on;
//   ia_gla_chunked      the same for portions of prompts cut into tiles of GLA_TILE rows that run side by side, behind
//                       a kernel that turns the portions' decay logits into decays once, in place: every
//                       tile but a request's last first runs from a zero state and leaves what it adds, U, and the
//                       product D of its decays; a second kernel walks a request's tiles, S <- diag(D) S + U, and
//                       leaves every tile the state before it; then every tile runs from that state and writes its
//                       rows, the last one the request's slot.  All of it fp32, as the recurrence itself;
//   ia_head_norm_gate   norm per head, weight, silu(gate), rounded once into the activations' type.
//
// The state of a head is kept in slices of GLA_PW value columns: slot[head][slice][n][GLA_PW], so that the workgroup
// that owns (request, head, slice) reads and writes one stretch of memory.  log(alpha) = log_sigmoid(z) / tau and
// every product that touches the state are fp32.
#include "common.h"

#define GLA_PW 16        // value columns of a workgroup's slice
#define GLA_PARTS 16     // the key channels are dealt out over so many groups of threads
#define GLA_TB 8         // tokens whose rows are staged together
#define GLA_TILE 64      // rows of a tile of ia_gla_chunked

__host__ __device__ inline int gla_slices(int vdim) { return (vdim + GLA_PW - 1) / GLA_PW; }

__device__ __forceinline__ float gla_log_sigmoid(float z) {
  // log(1 / (1 + exp(-z))): never above zero, no overflow on either side
  return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

// The record of the tile that begins at row r0 of request s: the tiles of the requests from ``first_request`` on,
// counted in the order of the requests and their rows, whatever the order of the list of tiles.
__device__ __forceinline__ int gla_record(const int* __restrict__ seq_starts, int first_request, int s, int r0) {
  int before = 0;
  for (int r = first_request; r < s; ++r) before += (seq_starts[r + 1] - seq_starts[r] + GLA_TILE - 1) / GLA_TILE;
  return before + r0 / GLA_TILE;
}

// grid (heads, requests or tiles, slices), 256 threads: thread (part, p) keeps S[n][p] for n = part, part + 16, ...
// in registers.  MODE 0: a request's rows from its slot, which is left moved on.  MODE 1: a tile (not a request's
// last) from a zero state; no rows are written, the state goes to the tile's record and the product of the decays
// to ``decay``.  MODE 2: a tile from its record; a request's last tile leaves the state in the slot.
template <typename T, int KMAX, int MODE>
__global__ __launch_bounds__(256) void gla_scan_kernel(
    const T* __restrict__ proj, int proj_stride, int q_col, int k_col, int v_col, const float* __restrict__ z,
    int z_stride, const float* __restrict__ z_bias, float inv_tau, float q_scale, float* __restrict__ state,
    long state_stride, float* __restrict__ out, const int* __restrict__ seq_starts, const int* __restrict__ state_slots,
    int nh, int dim, int vdim, const int* __restrict__ tiles, int first_request, float* __restrict__ records,
    long record_stride, float* __restrict__ decay, int form) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                                   // [TB][dim]
  float* ks = qs + GLA_TB * dim;                     // [TB][dim]
  float* as = ks + GLA_TB * dim;                     // [TB][dim]  alpha
  float* vs = as + GLA_TB * dim;                     // [TB][PW]
  float* ysum = vs + GLA_TB * GLA_PW;                // [TB][PARTS][PW]
  const int hd = blockIdx.x, slice = blockIdx.z;
  const int s = MODE == 0 ? blockIdx.y : tiles[2 * blockIdx.y];
  int first = seq_starts[s], count = seq_starts[s + 1] - first;
  bool last = true;
  int record = 0;
  if (MODE != 0) {
    const int r0 = tiles[2 * blockIdx.y + 1];
    last = r0 + GLA_TILE >= count;
    if (MODE == 2 || !last) record = gla_record(seq_starts, first_request, s, r0);
    first += r0;
    count = last ? count - r0 : GLA_TILE;
    if (MODE == 1 && last) return;
  }
  if (count <= 0) return;
  const int tid = threadIdx.x;
  const bool vec = (dim & 3) == 0;
  const int p = tid % GLA_PW, part = tid / GLA_PW;
  const int col = slice * GLA_PW + p;
  const int slices = gla_slices(vdim);
  const size_t within = ((size_t)hd * slices + slice) * dim * GLA_PW;
  float* S = state + (size_t)state_slots[s] * state_stride + within;
  float* R = MODE == 0 ? S : records + (size_t)record * record_stride + within;
  float dprod[MODE == 1 ? KMAX : 1];
  float reg[KMAX];
#pragma unroll
  for (int c = 0; c < KMAX; ++c) {
    const int n = part * KMAX + c;
    reg[c] = (MODE != 1 && n < dim) ? R[(size_t)n * GLA_PW + p] : 0.f;
    if constexpr (MODE == 1) dprod[c] = 1.f;
  }
  for (int t0 = 0; t0 < count; t0 += GLA_TB) {
    const int nt = count - t0 < GLA_TB ? count - t0 : GLA_TB;
    __syncthreads();                                  // the block before is read to its end
    for (int i = tid; i < nt * dim; i += 256) {
      const int t = i / dim, n = i - t * dim;
      const size_t row = (size_t)(first + t0 + t);
      const T* pr = proj + row * proj_stride;
      qs[i] = to_float(pr[q_col + hd * dim + n]) * q_scale;
      const float zz = z[row * z_stride + hd * dim + n];
      // the tiles read decays that one kernel made of the logits before them; the walk over a request makes its own.
      // form 1: z holds the decays themselves, and z_bias is no bias but the rows of fp32 keys that go with them
      // (what a channel takes in, 1 - decay, made where the decay was made and not as the difference of a number
      // near one), laid out like z
      const float a = (MODE != 0 || form == 1) ? zz : expf(gla_log_sigmoid(zz + (z_bias ? z_bias[hd * dim + n] : 0.f)) * inv_tau);
      as[i] = a;
      ks[i] = form == 1 ? z_bias[row * z_stride + hd * dim + n] : to_float(pr[k_col + hd * dim + n]);
    }
    for (int i = tid; i < nt * GLA_PW; i += 256) {
      const int t = i / GLA_PW, c = slice * GLA_PW + (i - t * GLA_PW);
      vs[i] = c < vdim ? to_float(proj[(size_t)(first + t0 + t) * proj_stride + v_col + hd * vdim + c]) : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float v = vs[t * GLA_PW + p];
      const float* qt = qs + t * dim;
      const float* kt = ks + t * dim;
      const float* at = as + t * dim;
      float acc = 0.f;
#pragma unroll
      for (int c4 = 0; c4 < KMAX; c4 += 4) {          // a thread's channels lie side by side: 16 bytes a read
        const int n0 = part * KMAX + c4;
        float a4[4], k4[4], q4[4];
        if (vec) {
          const bool in = n0 < dim;
          const float4 av = in ? *reinterpret_cast<const float4*>(at + n0) : make_float4(0.f, 0.f, 0.f, 0.f);
          const float4 kv = in ? *reinterpret_cast<const float4*>(kt + n0) : make_float4(0.f, 0.f, 0.f, 0.f);
          a4[0] = av.x; a4[1] = av.y; a4[2] = av.z; a4[3] = av.w;
          k4[0] = kv.x; k4[1] = kv.y; k4[2] = kv.z; k4[3] = kv.w;
          if (MODE != 1) {
            const float4 qv = in ? *reinterpret_cast<const float4*>(qt + n0) : make_float4(0.f, 0.f, 0.f, 0.f);
            q4[0] = qv.x; q4[1] = qv.y; q4[2] = qv.z; q4[3] = qv.w;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool in = n0 + e < dim;
            a4[e] = in ? at[n0 + e] : 0.f;
            k4[e] = in ? kt[n0 + e] : 0.f;
            q4[e] = (MODE != 1 && in) ? qt[n0 + e] : 0.f;
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {                  // channels past the head's last stay zero: 0 * 0 + 0 * v
          const int c = c4 + e;
          reg[c] = __builtin_fmaf(a4[e], reg[c], k4[e] * v);
          if constexpr (MODE == 1) dprod[c] *= a4[e];
          else acc = __builtin_fmaf(reg[c], q4[e], acc);
        }
      }
      if (MODE != 1) ysum[(t * GLA_PARTS + part) * GLA_PW + p] = acc;
    }
    if (MODE == 1) continue;
    __syncthreads();
    for (int i = tid; i < nt * GLA_PW; i += 256) {
      const int t = i / GLA_PW, pp = i - t * GLA_PW;
      const int c = slice * GLA_PW + pp;
      float y = ysum[(t * GLA_PARTS) * GLA_PW + pp];
#pragma unroll
      for (int k = 1; k < GLA_PARTS; ++k) y += ysum[(t * GLA_PARTS + k) * GLA_PW + pp];
      if (c < vdim) out[(size_t)(first + t0 + t) * ((size_t)nh * vdim) + (size_t)hd * vdim + c] = y;
    }
  }
  if (MODE == 2 && !last) return;
  float* W = MODE == 1 ? R : S;
#pragma unroll
  for (int c = 0; c < KMAX; ++c) {
    const int n = part * KMAX + c;
    if (n < dim) {
      W[(size_t)n * GLA_PW + p] = reg[c];
      if constexpr (MODE == 1) if (p == 0 && slice == 0) decay[((size_t)record * nh + hd) * dim + n] = dprod[c];
    }
  }
}

// grid (heads x slices x blocks of 256 values, tiles), 256 threads, a value of the state a thread; the workgroups of
// a request's first tile walk the request's tiles: the record of a tile holds what the tile adds when they come and
// the state before the tile when they go.  Eight tiles' loads are in flight together.
#define GLA_CHAIN_AHEAD 8
__global__ __launch_bounds__(256) void gla_chain_kernel(const float* __restrict__ state, long state_stride,
                                                        const int* __restrict__ seq_starts,
                                                        const int* __restrict__ state_slots, const int* __restrict__ tiles,
                                                        int first_request, float* __restrict__ records, long record_stride,
                                                        const float* __restrict__ decay, int nh, int dim, int slices) {
  const int i = blockIdx.y;
  if (tiles[2 * i + 1] != 0) return;
  const int s = tiles[2 * i], rows = seq_starts[s + 1] - seq_starts[s];
  const int per = (dim * GLA_PW + 255) / 256;
  const int hs = blockIdx.x / per, e = (blockIdx.x - hs * per) * 256 + threadIdx.x;
  if (e >= dim * GLA_PW) return;
  const int hd = hs / slices, n = e / GLA_PW;
  const size_t within = (size_t)hs * dim * GLA_PW + e;
  const int first = gla_record(seq_starts, first_request, s, 0);
  const int count = (rows + GLA_TILE - 1) / GLA_TILE;
  float S = state[(size_t)state_slots[s] * state_stride + within];
  for (int j0 = 0; j0 < count; j0 += GLA_CHAIN_AHEAD) {
    float U[GLA_CHAIN_AHEAD], D[GLA_CHAIN_AHEAD];
#pragma unroll
    for (int a = 0; a < GLA_CHAIN_AHEAD; ++a) {
      const int j = j0 + a;
      const bool adds = j < count - 1;                       // a request's last tile adds nothing that anyone reads
      U[a] = adds ? records[(size_t)(first + j) * record_stride + within] : 0.f;
      D[a] = adds ? decay[((size_t)(first + j) * nh + hd) * dim + n] : 0.f;
    }
#pragma unroll
    for (int a = 0; a < GLA_CHAIN_AHEAD; ++a) {
      const int j = j0 + a;
      if (j < count) {
        records[(size_t)(first + j) * record_stride + within] = S;
        if (j < count - 1) S = __builtin_fmaf(D[a], S, U[a]);
      }
    }
  }
}

// Floats a request's slot holds for one layer run.
extern "C" long ia_gla_state_floats(int nh, int dim, int vdim) { return (long)nh * gla_slices(vdim) * dim * GLA_PW; }

// proj: rows of proj_stride values (code: their type) holding q (nh dim values from q_col), k (from k_col) and v (nh vdim
// from v_col); z fp32 rows of z_stride values, z_bias (nullable) fp32 [nh dim]; out fp32 [N, nh vdim].
static int gla_scan_launch(const void* proj, int code, int proj_stride, int q_col, int k_col, int v_col, const float* z,
                           int z_stride, const float* z_bias, float tau, float q_scale, float* state, long state_stride,
                           float* out, const int* seq_starts, const int* state_slots, int B, int nh, int dim, int vdim,
                           int form, hipStream_t stream) {
  if (B == 0) return IA_OK;
  if (!proj || !z || !state || !out || !seq_starts || !state_slots || B < 0 || nh <= 0 || dim <= 0 || vdim <= 0 ||
      !(tau > 0.f) || q_col < 0 || k_col < 0 || v_col < 0 || proj_stride < q_col + nh * dim ||
      proj_stride < k_col + nh * dim || proj_stride < v_col + nh * vdim || z_stride < nh * dim ||
      state_stride < ia_gla_state_floats(nh, dim, vdim))
    return IA_ERR_BAD_ARG;
  const int per = (dim + GLA_PARTS - 1) / GLA_PARTS;
  const int slices = gla_slices(vdim);
  if (per > 32 || B > 65535 || slices > 65535) return IA_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)nh, (unsigned)B, (unsigned)slices);
  const size_t lds = sizeof(float) * ((size_t)3 * GLA_TB * dim + GLA_TB * GLA_PW + (size_t)GLA_TB * GLA_PARTS * GLA_PW);
  if (lds > 64 * 1024) return IA_ERR_UNSUPPORTED;
#define IA_GLA(T, KM)                                                                                                  \
  gla_scan_kernel<T, KM, 0><<<grid, 256, lds, stream>>>((const T*)proj, proj_stride, q_col, k_col, v_col, z, z_stride, \
                                                        z_bias, 1.0f / tau, q_scale, state, state_stride, out,         \
                                                        seq_starts, state_slots, nh, dim, vdim, nullptr, 0, nullptr,   \
                                                        0, nullptr, form)
#define IA_GLA_K(T)                       \
  do {                                    \
    if (per <= 4) IA_GLA(T, 4);           \
    else if (per <= 8) IA_GLA(T, 8);      \
    else if (per <= 16) IA_GLA(T, 16);    \
    else IA_GLA(T, 32);                   \
  } while (0)
  if (code == IA_F32) IA_GLA_K(float);
  else if (code == IA_BF16) IA_GLA_K(bf16_t);
  else return IA_ERR_BAD_ARG;
#undef IA_GLA_K
#undef IA_GLA
  IA_LAUNCH_CHECK();
  return IA_OK;
}

extern "C" int ia_gla_scan(const void* proj, int code, int proj_stride, int q_col, int k_col, int v_col, const float* z,
                           int z_stride, const float* z_bias, float tau, float q_scale, float* state, long state_stride,
                           float* out, const int* seq_starts, const int* state_slots, int B, int nh, int dim, int vdim,
                           hipStream_t stream) {
  return gla_scan_launch(proj, code, proj_stride, q_col, k_col, v_col, z, z_stride, z_bias, tau, q_scale, state,
                         state_stride, out, seq_starts, state_slots, B, nh, dim, vdim, 0, stream);
}

// The same recurrence with the decays given (f fp32 rows of f_stride values, each in [0, 1]) and the keys with them
// (k fp32, laid out like f: 1 - f, what a channel takes in because it does not keep it).  No factor on the queries.
extern "C" int ia_hgrn2_scan(const void* proj, int code, int proj_stride, int q_col, int v_col, const float* f,
                             const float* k, int f_stride, float* state, long state_stride, float* out,
                             const int* seq_starts, const int* state_slots, int B, int nh, int dim, int vdim,
                             hipStream_t stream) {
  if (!k) return IA_ERR_BAD_ARG;
  return gla_scan_launch(proj, code, proj_stride, q_col, q_col, v_col, f, f_stride, k, 1.0f, 1.0f, state,
                         state_stride, out, seq_starts, state_slots, B, nh, dim, vdim, 1, stream);
}

// z <- alpha = exp(log_sigmoid(z + bias) / tau) in place, for the rows from request ``first_request``'s first on.
__global__ __launch_bounds__(256) void gla_decays_kernel(float* __restrict__ z, int z_stride, const float* __restrict__ z_bias,
                                                         float inv_tau, const int* __restrict__ seq_starts,
                                                         int first_request, int num_rows, int cols) {
  const int row0 = seq_starts[first_request];
  const size_t total = (size_t)(num_rows - row0) * cols, stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const size_t r = i / cols;
    const int c = (int)(i - r * cols);
    float* at = z + (row0 + r) * z_stride + c;
    *at = expf(gla_log_sigmoid(*at + (z_bias ? z_bias[c] : 0.f)) * inv_tau);
  }
}

// The recurrence of ia_gla_scan for the requests that the tiles name: tiles[i] = (request, first row of a tile of
// GLA_TILE among the request's rows) in any order, every tile of the requests first_request .. (and of no other)
// once.  records: fp32 [num_tiles, record_stride >= ia_gla_state_floats]; decay: fp32 [num_tiles, nh, dim].  z has
// num_rows rows; those of the requests first_request .. are left holding the decays, not the logits.
static int gla_chunked_launch(const void* proj, int code, int proj_stride, int q_col, int k_col, int v_col, const float* z,
                              int z_stride, const float* z_bias, float tau, float q_scale, float* state,
                              long state_stride, float* out, const int* seq_starts, const int* state_slots,
                              const int* tiles, int num_tiles, int first_request, int num_rows, float* records, long record_stride, float* decay, int nh,
                              int dim, int vdim, int form, hipStream_t stream) {
  if (num_tiles == 0) return IA_OK;
  if (!proj || !z || !state || !out || !seq_starts || !state_slots || !tiles || !records || !decay || num_tiles < 0 || first_request < 0 || num_rows <= 0 ||
      nh <= 0 || dim <= 0 || vdim <= 0 || !(tau > 0.f) || q_col < 0 || k_col < 0 || v_col < 0 ||
      proj_stride < q_col + nh * dim || proj_stride < k_col + nh * dim || proj_stride < v_col + nh * vdim ||
      z_stride < nh * dim || state_stride < ia_gla_state_floats(nh, dim, vdim) ||
      record_stride < ia_gla_state_floats(nh, dim, vdim))
    return IA_ERR_BAD_ARG;
  const int per = (dim + GLA_PARTS - 1) / GLA_PARTS;
  const int slices = gla_slices(vdim);
  if (per > 32 || num_tiles > 65535 || slices > 65535) return IA_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)nh, (unsigned)num_tiles, (unsigned)slices);
  const size_t lds = sizeof(float) * ((size_t)3 * GLA_TB * dim + GLA_TB * GLA_PW + (size_t)GLA_TB * GLA_PARTS * GLA_PW);
  if (lds > 64 * 1024) return IA_ERR_UNSUPPORTED;
#define IA_GLA(T, KM, MODE)                                                                                        \
  gla_scan_kernel<T, KM, MODE><<<grid, 256, lds, stream>>>(                                                        \
      (const T*)proj, proj_stride, q_col, k_col, v_col, z, z_stride, z_bias, 1.0f / tau, q_scale, state,           \
      state_stride, out, seq_starts, state_slots, nh, dim, vdim, tiles, first_request, records, record_stride, decay, form)
#define IA_GLA_K(T, MODE)                       \
  do {                                          \
    if (per <= 4) IA_GLA(T, 4, MODE);           \
    else if (per <= 8) IA_GLA(T, 8, MODE);      \
    else if (per <= 16) IA_GLA(T, 16, MODE);    \
    else IA_GLA(T, 32, MODE);                   \
  } while (0)
#define IA_GLA_T(MODE)                             \
  do {                                             \
    if (code == IA_F32) IA_GLA_K(float, MODE);     \
    else IA_GLA_K(bf16_t, MODE);                   \
  } while (0)
  if (code != IA_F32 && code != IA_BF16) return IA_ERR_BAD_ARG;
  if (form == 0) {
    const size_t most = (size_t)num_rows * nh * dim;
    gla_decays_kernel<<<(unsigned)((most + 255) / 256 < 262144 ? (most + 255) / 256 : 262144), 256, 0, stream>>>(
        const_cast<float*>(z), z_stride, z_bias, 1.0f / tau, seq_starts, first_request, num_rows, nh * dim);
    IA_LAUNCH_CHECK();
  }
  IA_GLA_T(1);
  IA_LAUNCH_CHECK();
  gla_chain_kernel<<<dim3((unsigned)(nh * slices * ((dim * GLA_PW + 255) / 256)), (unsigned)num_tiles), 256, 0, stream>>>(
      state, state_stride, seq_starts, state_slots, tiles, first_request, records, record_stride, decay, nh, dim, slices);
  IA_LAUNCH_CHECK();
  IA_GLA_T(2);
#undef IA_GLA_T
#undef IA_GLA_K
#undef IA_GLA
  IA_LAUNCH_CHECK();
  return IA_OK;
}

extern "C" int ia_gla_chunked(const void* proj, int code, int proj_stride, int q_col, int k_col, int v_col, const float* z,
                              int z_stride, const float* z_bias, float tau, float q_scale, float* state,
                              long state_stride, float* out, const int* seq_starts, const int* state_slots,
                              const int* tiles, int num_tiles, int first_request, int num_rows, float* records, long record_stride, float* decay, int nh,
                              int dim, int vdim, hipStream_t stream) {
  return gla_chunked_launch(proj, code, proj_stride, q_col, k_col, v_col, z, z_stride, z_bias, tau, q_scale, state,
                            state_stride, out, seq_starts, state_slots, tiles, num_tiles, first_request, num_rows, records,
                            record_stride, decay, nh, dim, vdim, 0, stream);
}

// ia_gla_chunked with the decays and the keys given (see ia_hgrn2_scan); f is left as it is.
extern "C" int ia_hgrn2_chunked(const void* proj, int code, int proj_stride, int q_col, int v_col, const float* f,
                                const float* k, int f_stride, float* state, long state_stride, float* out, const int* seq_starts,
                                const int* state_slots, const int* tiles, int num_tiles, int first_request, int num_rows,
                                float* records, long record_stride, float* decay, int nh, int dim, int vdim,
                                hipStream_t stream) {
  if (!k) return IA_ERR_BAD_ARG;
  return gla_chunked_launch(proj, code, proj_stride, q_col, q_col, v_col, f, f_stride, k, 1.0f, 1.0f, state,
                            state_stride, out, seq_starts, state_slots, tiles, num_tiles, first_request, num_rows, records,
                            record_stride, decay, nh, dim, vdim, 1, stream);
}

// The gates of that recurrence: the q columns of proj become silu(q) in place (in the activations' type), z (fp32
// [N, cols], the logits of the forget gate) becomes f = lower + (1 - lower) sigmoid(z + bias) in place, and k (laid
// out like z) gets 1 - f = (1 - lower) sigmoid(-(z + bias)), which is exact where f is within rounding of one.
template <typename T>
__global__ __launch_bounds__(256) void hgrn2_gates_kernel(T* __restrict__ proj, int proj_stride, int q_col,
                                                          float* __restrict__ z, float* __restrict__ k, int z_stride,
                                                          const float* __restrict__ bias, const float* __restrict__ lower,
                                                          long total, int cols) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const long n = i / cols;
  const int c = (int)(i - n * cols);
  T* q = proj + (size_t)n * proj_stride + q_col + c;
  const float qv = to_float(*q);
  *q = from_float<T>(qv / (1.0f + expf(-qv)));
  float* zz = z + (size_t)n * z_stride + c;
  const float lo = lower ? lower[c] : 0.f;
  const float x = *zz + (bias ? bias[c] : 0.f);
  *zz = lo + (1.0f - lo) * (1.0f / (1.0f + expf(-x)));
  k[(size_t)n * z_stride + c] = (1.0f - lo) * (1.0f / (1.0f + expf(x)));
}

extern "C" int ia_hgrn2_gates(void* proj, int code, int proj_stride, int q_col, float* z, float* k, int z_stride,
                              const float* bias, const float* lower, int N, int cols, hipStream_t stream) {
  if (N < 0 || cols <= 0 || q_col < 0 || proj_stride < q_col + cols || z_stride < cols) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!proj || !z || !k) return IA_ERR_BAD_ARG;
  const long total = (long)N * cols;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (code == IA_F32)
    hgrn2_gates_kernel<float><<<grid, 256, 0, stream>>>((float*)proj, proj_stride, q_col, z, k, z_stride, bias, lower, total, cols);
  else if (code == IA_BF16)
    hgrn2_gates_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)proj, proj_stride, q_col, z, k, z_stride, bias, lower, total, cols);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// One wave per (token, head): y = o / sqrt(mean(o^2) + eps) * w * silu(gate), o fp32 [N, nh vdim], w fp32 [vdim],
// gate rows of gate_stride values in the activations' type (the head's vdim values from gate_col + head * vdim).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                             int gate_stride, int gate_col, const float* __restrict__ w,
                                                             T* __restrict__ y, long pairs, int nh, int vdim, float eps) {
  const long pair = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long n = pair / nh;
  const int hd = (int)(pair - n * nh);
  const float* orow = o + (size_t)pair * vdim;
  float ss = 0.f;
  for (int i = lane; i < vdim; i += 64) ss = fmaf(orow[i], orow[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
  if (!gate) {                       // no gate: the norm and the weight alone
    for (int i = lane; i < vdim; i += 64) y[(size_t)pair * vdim + i] = from_float<T>(orow[i] * inv * w[i]);
    return;
  }
  const T* grow = gate + (size_t)n * gate_stride + gate_col + (size_t)hd * vdim;
  for (int i = lane; i < vdim; i += 64) {
    const float g = to_float(grow[i]);
    y[(size_t)pair * vdim + i] = from_float<T>(orow[i] * inv * w[i] * (g / (1.0f + expf(-g))));
  }
}

extern "C" int ia_head_norm_gate(const float* o, const void* gate, int code, int gate_stride, int gate_col,
                                 const float* w, void* y, int N, int nh, int vdim, float eps, hipStream_t stream) {
  if (N < 0 || nh <= 0 || vdim <= 0 || !(eps > 0.f) || (gate && (gate_col < 0 || gate_stride < gate_col + nh * vdim)))
    return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!o || !w || !y) return IA_ERR_BAD_ARG;
  const long pairs = (long)N * nh;
  const long blocks = (pairs + 3) / 4;
  if (blocks > 0x7fffffffL) return IA_ERR_UNSUPPORTED;
  if (code == IA_F32)
    head_norm_gate_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(o, (const float*)gate, gate_stride, gate_col, w,
                                                                       (float*)y, pairs, nh, vdim, eps);
  else if (code == IA_BF16)
    head_norm_gate_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(o, (const bf16_t*)gate, gate_stride, gate_col, w,
                                                                        (bf16_t*)y, pairs, nh, vdim, eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_gla_scan)
IA_OP(ia_gla_chunked)
IA_OP(ia_hgrn2_scan)
IA_OP(ia_hgrn2_chunked)
IA_OP(ia_hgrn2_gates)
IA_OP(ia_head_norm_gate)
