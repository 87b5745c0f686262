// Attention with sigmoid weights over the paged cache on the matrix cores (v_mfma_f32_16x16x16_bf16), compiled for
// one pair of head sizes: SA_DIM values a key, SA_VDIM a value (multiples of 16, at most 256).
//
//     w_ij = sigmoid( scale q_i.k_j - r1_h ln(1 + r2_h (i - j)) + b_h )   for j <= i,      o_i = g_ih sum_j w_ij v_j
//
// Both kernels work on the transposed problem, 16 keys against 16 columns at a time:
//     S^T[key, col] = K[key, :] . Q[col, :]            A operand: 16 keys, B operand: 16 columns of queries
//     O^T[c, col]  += V^T[c, key] W^T[key, col]        A operand: 16 value channels x 4 keys, B operand: the weights
// The accumulator of S^T leaves lane l with the keys 4 (l / 16) .. + 3 of column l % 16, which is what the B operand
// of the second product wants, so the weights go from registers to registers (rounded to bf16; their scores, the
// distance term and the sigmoid are fp32).  Value pages are transposed, [num_pages, nkv, vdim, page_size], so that
// the A operand of the second product is 8 contiguous bytes; key pages are [num_pages, nkv, page_size, dim].  The
// page size is a multiple of 4.  A sum of sigmoids has no maximum to follow and nothing to rescale: partial sums over
// parts of the keys simply add up, in a fixed order.
//
// Single tokens: the 16 columns are up to 16 query heads of ONE key/value head of one token, so a page is read once
// for its group of heads; the keys are split over blockIdx.z and over the four waves of a workgroup (every fourth
// tile of 16 keys); the waves join through LDS, the parts through fp32 records and a second small kernel.
// Portions of prompts: a wave takes 16 consecutive rows of one query head; a workgroup 64 rows (a tile the host lists).
//
// Values of keys that no column of the tile sees are zeroed after the load and their weights are zero: a stale or
// poisoned page never leaks in.  A key that is needed but has no page in the block table gives NaN, not a fault.
#include "common.h"

#ifndef SA_DIM
#error "compile with -DSA_DIM=<key size> -DSA_VDIM=<value size>"
#endif
#define NSK (SA_DIM / 16)
#define NSV (SA_VDIM / 16)
static_assert(SA_DIM % 16 == 0 && SA_DIM >= 16 && SA_DIM <= 256, "key size: a multiple of 16 up to 256");
static_assert(SA_VDIM % 16 == 0 && SA_VDIM >= 16 && SA_VDIM <= 256, "value size: a multiple of 16 up to 256");

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ s16x4 sa_s16x4(uint32_t a, uint32_t b) {
  uint2 u = make_uint2(a, b);
  return __builtin_bit_cast(s16x4, u);
}

// The NSK steps' worth of one row (a key, or a column of queries) for lane group qd: step s covers the values
// (s / 2) 32 + qd 8 + (s % 2) 4 .. + 3 (16-byte loads); an odd last step covers (SA_DIM / 32) 32 + qd 4 .. + 3.
// Keys and queries use the same map, and a dot product does not care about the order of its terms.
__device__ __forceinline__ void sa_load_row(const uint16_t* __restrict__ row, int qd, s16x4 (&reg)[NSK]) {
#pragma unroll
  for (int t = 0; t < SA_DIM / 32; ++t) {
    const uint4 v = *reinterpret_cast<const uint4*>(row + t * 32 + qd * 8);
    reg[2 * t] = sa_s16x4(v.x, v.y);
    reg[2 * t + 1] = sa_s16x4(v.z, v.w);
  }
  if (SA_DIM % 32) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + (SA_DIM / 32) * 32 + qd * 4);
    reg[NSK - 1] = sa_s16x4(v.x, v.y);
  }
}

struct SaGeom {
  const uint16_t* k_base;        // pages of this key/value head
  const uint16_t* v_base;
  const int* bt;                 // the request's row of the block table
  size_t k_page, v_page;         // values from a page to the next
  int ps, ps_shift, num_pages;
};

struct SaHead {                  // the numbers of this lane's column (a head)
  float scale, bias, c2, a2;     // score scale + bias + c2 log2(1 + a2 distance),  c2 = -r1 ln 2
};

// One tile of 16 keys, t0 .. t0 + 15, against the wave's 16 columns.  ``pos``: the last key this lane's column sees
// (below zero: no such column); ``kmax``: the last key any column of the wave sees (the same in all lanes).
// POW2: the page size is a power of two (a shift and a mask instead of a division by a number known at run time).
template <bool POW2>
__device__ __forceinline__ void sa_tile(const SaGeom& G, const SaHead& H, int t0, int j, int qd, int pos, int kmax,
                                        const s16x4 (&q)[NSK], f32x4 (&o)[NSV], bool& bad) {
  // ---- loads: this lane's key row, and four keys' values of NSV channels
  const int key = t0 + j;
  const int keyc = key > kmax ? kmax : key;
  const int page = G.bt[POW2 ? keyc >> G.ps_shift : keyc / G.ps];
  const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
  s16x4 kr[NSK];
  sa_load_row(G.k_base + (size_t)(page_ok ? page : 0) * G.k_page + (size_t)(POW2 ? keyc & (G.ps - 1) : keyc % G.ps) * SA_DIM, qd, kr);
  const int kg = t0 + 4 * qd;    // this lane brings the values of the keys kg .. kg + 3 (one quad, one page)
  const int kgc = kg > kmax ? (kmax & ~3) : kg;
  const int pagev = G.bt[POW2 ? kgc >> G.ps_shift : kgc / G.ps];
  const bool pagev_ok = (unsigned)pagev < (unsigned)G.num_pages;
  const uint16_t* vq = G.v_base + (size_t)(pagev_ok ? pagev : 0) * G.v_page + (POW2 ? kgc & (G.ps - 1) : kgc % G.ps);
  uint2 v[NSV];
#pragma unroll
  for (int n = 0; n < NSV; ++n) v[n] = *reinterpret_cast<const uint2*>(vq + (size_t)(n * 16 + j) * G.ps);
  uint32_t mlo = 0u, mhi = 0u;
  if (kg == kgc && pagev_ok) {
    mlo = (kg <= kmax ? 0x0000ffffu : 0u) | (kg + 1 <= kmax ? 0xffff0000u : 0u);
    mhi = (kg + 2 <= kmax ? 0x0000ffffu : 0u) | (kg + 3 <= kmax ? 0xffff0000u : 0u);
  }
  bad = bad || (key <= kmax && !page_ok) || (kg <= kmax && !pagev_ok);
  // ---- S^T = K Q^T
  f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < NSK; ++st) s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kr[st], q[st], s, 0, 0, 0);
  // ---- the weights of this lane's four keys, fp32, then rounded once as the operand of the second product
  float w[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int kk = kg + r;
    const float dist = (float)(pos - kk);
    const float x = fmaf(s[r], H.scale, H.bias) + H.c2 * __builtin_amdgcn_logf(fmaf(H.a2, dist, 1.0f));
    const float e = __builtin_amdgcn_exp2f(-1.4426950408889634f * x);
    w[r] = kk <= pos ? __builtin_amdgcn_rcpf(1.0f + e) : 0.f;
  }
  const f32x2_t w0 = {w[0], w[1]}, w1 = {w[2], w[3]};
  const uint32_t p0 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w0, bf16x2_t));
  const uint32_t p1 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w1, bf16x2_t));
  const s16x4 pw = sa_s16x4(p0, p1);
  // ---- O^T += V^T W^T
#pragma unroll
  for (int n = 0; n < NSV; ++n)
    o[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(sa_s16x4(v[n].x & mlo, v[n].y & mhi), pw, o[n], 0, 0, 0);
}

__device__ __forceinline__ SaHead sa_head(const float* r1, const float* r2, const float* pb, int h, float scale) {
  SaHead H;
  H.scale = scale;
  H.bias = pb ? pb[h] : 0.f;
  H.c2 = r1 ? -0.6931471805599453f * r1[h] : 0.f;
  H.a2 = r2 ? r2[h] : 0.f;
  return H;
}

__device__ __forceinline__ float sa_gate(const uint16_t* gate, size_t at) {
  return gate ? 1.0f / (1.0f + expf(-bf16_bits_to_float(gate[at]))) : 1.0f;
}

__device__ __forceinline__ void sa_store_bf16x4(uint16_t* at, const f32x4& x, float f) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(x[0] * f) | ((uint32_t)float_to_bf16_bits(x[1] * f) << 16);
  u.y = (uint32_t)float_to_bf16_bits(x[2] * f) | ((uint32_t)float_to_bf16_bits(x[3] * f) << 16);
  *reinterpret_cast<uint2*>(at) = u;
}

// ------------------------------------------------------------------------ single tokens
// grid (B, nkv * ceil(G / 16), parts), 256 threads.  Token b is row b of q, gate and out and of the block tables.
// parts == 1: out is written (gated, bf16); otherwise records part[(b parts + z) nh + h][SA_VDIM] of fp32.
template <bool POW2>
__global__ __launch_bounds__(256) void sigattn_decode_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const uint16_t* __restrict__ gate, int gate_stride, uint16_t* __restrict__ out,
    float* __restrict__ part, const int* __restrict__ positions, const int* __restrict__ block_tables, int bt_stride,
    const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ pb, int nh, int nkv, int ps,
    int num_pages, float scale, int parts) {
  __shared__ f32x4 red[3][NSV][64];
  __shared__ int s_bad;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, qd = lane >> 4;
  const int b = blockIdx.x, z = blockIdx.z;
  const int Gq = nh / nkv, HC = (Gq + 15) / 16;
  const int g = blockIdx.y / HC, hc = blockIdx.y - g * HC;
  const int hj = hc * 16 + j;
  const bool col_ok = hj < Gq;
  const int h = g * Gq + (col_ok ? hj : 0);
  const int p = positions[b];
  if (tid == 0) s_bad = 0;
  SaGeom G;
  G.k_page = (size_t)nkv * ps * SA_DIM;
  G.v_page = (size_t)nkv * ps * SA_VDIM;
  G.k_base = k_pages + (size_t)g * ps * SA_DIM;
  G.v_base = v_pages + (size_t)g * ps * SA_VDIM;
  G.bt = block_tables + (size_t)b * bt_stride;
  G.ps = ps;
  G.ps_shift = 31 - __clz(ps);
  G.num_pages = num_pages;
  const SaHead H = sa_head(r1, r2, pb, h, scale);
  s16x4 qr[NSK];
  sa_load_row(q + (size_t)b * q_stride + (size_t)h * SA_DIM, qd, qr);
  f32x4 o[NSV];
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  bool bad = false;
  const int tiles = p / 16 + 1, per = (tiles + parts - 1) / parts;
  const int tbeg = z * per, tend = tbeg + per < tiles ? tbeg + per : tiles;
  const int pos = col_ok ? p : -1;
  for (int t = tbeg + wave; t < tend; t += 4) sa_tile<POW2>(G, H, t * 16, j, qd, pos, p, qr, o, bad);
  __syncthreads();
  if (bad) s_bad = 1;
  if (wave > 0) {
#pragma unroll
    for (int n = 0; n < NSV; ++n) red[wave - 1][n][lane] = o[n];
  }
  __syncthreads();
  if (wave > 0 || !col_ok) return;
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = ((o[n] + red[0][n][lane]) + red[1][n][lane]) + red[2][n][lane];
  if (s_bad) {
#pragma unroll
    for (int n = 0; n < NSV; ++n) o[n][0] = o[n][1] = o[n][2] = o[n][3] = __uint_as_float(0x7fc00000u);
  }
  if (parts == 1) {
    const float gt = sa_gate(gate, (size_t)b * gate_stride + h);
    uint16_t* at = out + ((size_t)b * nh + h) * SA_VDIM + 4 * qd;
#pragma unroll
    for (int n = 0; n < NSV; ++n) sa_store_bf16x4(at + n * 16, o[n], gt);
  } else {
    float* at = part + (((size_t)b * parts + z) * nh + h) * SA_VDIM + 4 * qd;
#pragma unroll
    for (int n = 0; n < NSV; ++n) *reinterpret_cast<f32x4*>(at + n * 16) = o[n];
  }
}

// grid (B, nh), 64 threads: the parts of a token's head added in their order, gated, rounded once.
__global__ __launch_bounds__(64) void sigattn_join_kernel(const float* __restrict__ part, const uint16_t* __restrict__ gate,
                                                          int gate_stride, uint16_t* __restrict__ out, int nh, int parts) {
  const int b = blockIdx.x, h = blockIdx.y;
  const float gt = sa_gate(gate, (size_t)b * gate_stride + h);
  for (int c = threadIdx.x; c < SA_VDIM; c += 64) {
    float acc = 0.f;
    for (int z = 0; z < parts; ++z) acc += part[(((size_t)b * parts + z) * nh + h) * SA_VDIM + c];
    out[((size_t)b * nh + h) * SA_VDIM + c] = float_to_bf16_bits(acc * gt);
  }
}

// ------------------------------------------------------------------------ portions of prompts
// 256 threads; a workgroup is one tile (request, first row) of 64 rows and one query head; wave w takes the rows
// first + 16 w .. + 15.  Workgroups are numbered so that the heads of one tile follow each other (they go to
// different dies, each of which then keeps its heads' keys in its L2), the tiles in the order of the host's list
// (which puts those with the most keys first).
template <bool POW2>
__global__ __launch_bounds__(256) void sigattn_prefill_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const uint16_t* __restrict__ gate, int gate_stride, uint16_t* __restrict__ out,
    const int* __restrict__ seq_starts, const int* __restrict__ seq_ctx, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ tiles, int num_tiles, const float* __restrict__ r1,
    const float* __restrict__ r2, const float* __restrict__ pb, int nh, int nkv, int ps, int num_pages, float scale) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, qd = lane >> 4;
  const int lin = blockIdx.x;
  const int tile = lin / nh, h = lin - tile * nh;
  const int sidx = tiles[2 * tile], row0 = tiles[2 * tile + 1];
  const int qstart = seq_starts[sidx], qlen = seq_starts[sidx + 1] - qstart, ctx = seq_ctx[sidx];
  const int rb = row0 + wave * 16;
  if (rb >= qlen) return;                                   // the waves share nothing: no barrier follows
  const int g = h / (nh / nkv);
  const int row = rb + j;
  const bool col_ok = row < qlen;
  const int pos = col_ok ? ctx + row : -1;
  const int kmax = ctx + (rb + 15 < qlen ? rb + 15 : qlen - 1);
  SaGeom G;
  G.k_page = (size_t)nkv * ps * SA_DIM;
  G.v_page = (size_t)nkv * ps * SA_VDIM;
  G.k_base = k_pages + (size_t)g * ps * SA_DIM;
  G.v_base = v_pages + (size_t)g * ps * SA_VDIM;
  G.bt = block_tables + (size_t)sidx * bt_stride;
  G.ps = ps;
  G.ps_shift = 31 - __clz(ps);
  G.num_pages = num_pages;
  const SaHead H = sa_head(r1, r2, pb, h, scale);
  const size_t qrow = (size_t)(qstart + (col_ok ? row : rb));
  s16x4 qr[NSK];
  sa_load_row(q + qrow * q_stride + (size_t)h * SA_DIM, qd, qr);
  f32x4 o[NSV];
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  bool bad = false;
  for (int t0 = 0; t0 <= kmax; t0 += 16) sa_tile<POW2>(G, H, t0, j, qd, pos, kmax, qr, o, bad);
  if (__any(bad)) {
#pragma unroll
    for (int n = 0; n < NSV; ++n) o[n][0] = o[n][1] = o[n][2] = o[n][3] = __uint_as_float(0x7fc00000u);
  }
  if (!col_ok) return;
  const float gt = sa_gate(gate, qrow * gate_stride + h);
  uint16_t* at = out + (qrow * nh + h) * SA_VDIM + 4 * qd;
#pragma unroll
  for (int n = 0; n < NSV; ++n) sa_store_bf16x4(at + n * 16, o[n], gt);
}

// ------------------------------------------------------------------------ launchers
extern "C" int ia_sigattn_dim() { return SA_DIM; }
extern "C" int ia_sigattn_vdim() { return SA_VDIM; }

static int sa_check(int nh, int nkv, int ps, int num_pages, int bt_stride, int q_stride, const void* gate,
                    int gate_stride) {
  if (nh <= 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || (ps & 3) || num_pages <= 0 || bt_stride <= 0 ||
      q_stride < nh * SA_DIM || (gate && gate_stride < nh))
    return IA_ERR_BAD_ARG;
  if (q_stride & 7) return IA_ERR_UNSUPPORTED;              // 16-byte loads of the queries
  return IA_OK;
}

// q rows of q_stride bf16 values (head h's SA_DIM values from h SA_DIM); gate (nullable): rows of gate_stride values,
// head h's logit at [h]; out [B, nh SA_VDIM] bf16; part: parts > 1 only, fp32 [B parts nh SA_VDIM].
extern "C" int ia_sigattn_decode(const void* q, int q_stride, const void* k_pages, const void* v_pages, const void* gate,
                                 int gate_stride, void* out, float* part, const int* positions, const int* block_tables,
                                 int bt_stride, const float* r1, const float* r2, const float* pb, int B, int nh, int nkv,
                                 int ps, int num_pages, float scale, int parts, hipStream_t stream) {
  if (B < 0 || parts < 1 || parts > 65535 || (parts > 1 && !part)) return IA_ERR_BAD_ARG;
  const int rc = sa_check(nh, nkv, ps, num_pages, bt_stride, q_stride, gate, gate_stride);
  if (rc != IA_OK) return rc;
  if (B == 0) return IA_OK;
  const int HC = (nh / nkv + 15) / 16;
  if ((long long)nkv * HC > 65535 || nh > 65535) return IA_ERR_UNSUPPORTED;
  dim3 grid(B, nkv * HC, parts);
#define SA_DEC(P2)                                                                                               \
  sigattn_decode_kernel<P2><<<grid, 256, 0, stream>>>(                                                           \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, (const uint16_t*)gate,   \
      gate_stride, (uint16_t*)out, part, positions, block_tables, bt_stride, r1, r2, pb, nh, nkv, ps, num_pages, \
      scale, parts)
  if ((ps & (ps - 1)) == 0) SA_DEC(true);
  else SA_DEC(false);
#undef SA_DEC
  IA_LAUNCH_CHECK();
  if (parts > 1) {
    sigattn_join_kernel<<<dim3(B, nh), 64, 0, stream>>>(part, (const uint16_t*)gate, gate_stride, (uint16_t*)out, nh,
                                                        parts);
    IA_LAUNCH_CHECK();
  }
  return IA_OK;
}

// tiles[i] = (request, first row of a tile of 64 among the request's rows); request s has the rows
// seq_starts[s] .. seq_starts[s + 1] - 1 of q, gate and out, seq_ctx[s] keys before its first row, and row s of
// the block tables.
extern "C" int ia_sigattn_prefill(const void* q, int q_stride, const void* k_pages, const void* v_pages, const void* gate,
                                  int gate_stride, void* out, const int* seq_starts, const int* seq_ctx,
                                  const int* block_tables, int bt_stride, const int* tiles, int num_tiles,
                                  const float* r1, const float* r2, const float* pb, int nh, int nkv, int ps,
                                  int num_pages, float scale, hipStream_t stream) {
  if (num_tiles < 0) return IA_ERR_BAD_ARG;
  const int rc = sa_check(nh, nkv, ps, num_pages, bt_stride, q_stride, gate, gate_stride);
  if (rc != IA_OK) return rc;
  if (num_tiles == 0) return IA_OK;
  if (!tiles || !seq_starts || !seq_ctx) return IA_ERR_BAD_ARG;
  if ((long long)num_tiles * nh > 0x7fffffffLL) return IA_ERR_UNSUPPORTED;
#define SA_PRE(P2)                                                                                                \
  sigattn_prefill_kernel<P2><<<num_tiles * nh, 256, 0, stream>>>(                                                 \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, (const uint16_t*)gate,    \
      gate_stride, (uint16_t*)out, seq_starts, seq_ctx, block_tables, bt_stride, tiles, num_tiles, r1, r2, pb, nh, \
      nkv, ps, num_pages, scale)
  if ((ps & (ps - 1)) == 0) SA_PRE(true);
  else SA_PRE(false);
#undef SA_PRE
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_sigattn_decode)
IA_OP(ia_sigattn_prefill)
