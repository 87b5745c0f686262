// Attention over a sliding window of keys and pooled blocks before it (window_pool_attention.hip has the rule and the
// plain kernels) on the matrix cores (v_mfma_f32_16x16x16_bf16), compiled for one pair of head sizes: WP_DIM values a
// key, WP_VDIM a value (multiples of 16, at most 256).
//
// Both kernels work on the transposed problem, 16 keys (or blocks) against 16 columns at a time:
//     S^T[key, col] = K[key, :] . Q[col, :]            A operand: 16 keys, B operand: 16 columns of queries
//     O^T[c, col]  += V^T[c, key] P^T[key, col]        A operand: 16 value channels x 4 keys, B operand: the weights
// The accumulator of S^T leaves lane l with the keys 4 (l / 16) .. + 3 of column l % 16, which is what the B operand
// of the second product wants, so the weights go from registers to registers (rounded to bf16; scores, maximum,
// exponentials and their sum are fp32, and the sum is taken of the rounded weights, so that numerator and
// denominator agree).  A column's running maximum is the same in its four lanes (two exchanges a tile); every lane
// keeps the sum of its own keys' weights, and the four meet at the end.
//
// Token pages: keys [num_pages, nkv, page_size, WP_DIM], values transposed [num_pages, nkv, WP_VDIM, page_size] (the A
// operand of the second product is then 8 contiguous bytes; the page size is a multiple of 4).  Pooled pages: keys
// [num_pages, nkv, E, WP_DIM], values [num_pages, nkv, E, WP_VDIM] with E = (page_size - 1) / P + 1: the entry of
// block b lies in the page of its last position t = b P + P - 1 at place (t % page_size) / P; neighbouring blocks need
// not be neighbours there, so a block's values are fetched one by one (there are few blocks: a position in P).
//
// The 16 columns are 16 consecutive rows of one query head (portions of prompts) or up to 16 query heads of one
// key/value head of one token (single tokens); the tiles (of blocks, then of keys) are dealt out over the four waves
// of a workgroup, which join through LDS in the order of the waves.
// Values of keys that no column of the tile sees are zeroed after the load and their weights are zero: a page that
// went back to the pool never leaks in.  A key that is needed but has no page in the block table gives NaN.
#include "common.h"

#ifndef WP_DIM
#error "compile with -DWP_DIM=<key size> -DWP_VDIM=<value size>"
#endif
#define NSK (WP_DIM / 16)
#define NSV (WP_VDIM / 16)
static_assert(WP_DIM % 16 == 0 && WP_DIM >= 16 && WP_DIM <= 256, "key size: a multiple of 16 up to 256");
static_assert(WP_VDIM % 16 == 0 && WP_VDIM >= 16 && WP_VDIM <= 256, "value size: a multiple of 16 up to 256");
#define WP_LOG2E 1.4426950408889634f

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ s16x4 wp_s16x4(uint32_t a, uint32_t b) {
  uint2 u = make_uint2(a, b);
  return __builtin_bit_cast(s16x4, u);
}

// The NSK steps' worth of one row (a key, or a column of queries) for lane group qd: step s covers the values
// (s / 2) 32 + qd 8 + (s % 2) 4 .. + 3 (16-byte loads); an odd last step covers (WP_DIM / 32) 32 + qd 4 .. + 3.
// Keys and queries use the same map, and a dot product does not care about the order of its terms.
__device__ __forceinline__ void wp_load_row(const uint16_t* __restrict__ row, int qd, s16x4 (&reg)[NSK]) {
#pragma unroll
  for (int t = 0; t < WP_DIM / 32; ++t) {
    const uint4 v = *reinterpret_cast<const uint4*>(row + t * 32 + qd * 8);
    reg[2 * t] = wp_s16x4(v.x, v.y);
    reg[2 * t + 1] = wp_s16x4(v.z, v.w);
  }
  if (WP_DIM % 32) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + (WP_DIM / 32) * 32 + qd * 4);
    reg[NSK - 1] = wp_s16x4(v.x, v.y);
  }
}

struct WpGeom {
  const uint16_t* k_base;        // token pages of this key/value head
  const uint16_t* v_base;
  const int* bt;                 // the request's row of the token pages' block table
  size_t k_page, v_page;         // values from a page to the next
  int ps, ps_shift, num_pages;
  const uint16_t* pk_base;       // pooled pages of this key/value head
  const uint16_t* pv_base;
  const int* btp;
  size_t pk_page, pv_page;
  int E, P, num_pool_pages;
};

struct WpCol {                   // what a lane keeps of its column
  float m, l;                    // running maximum (log2 domain, the same in the column's four lanes), own keys' sum
};

// The scores of this lane's four keys (``ok[r]``: the column sees key r) into the running softmax: the weights come
// back as the B operand of the second product.
__device__ __forceinline__ s16x4 wp_softmax_step(const f32x4& s, const bool (&ok)[4], float scale_log2, WpCol& c,
                                                 f32x4 (&o)[NSV]) {
  float x[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) x[r] = ok[r] ? s[r] * scale_log2 : -INFINITY;
  float tm = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
  tm = fmaxf(tm, __shfl_xor(tm, 16, IA_WAVE));
  tm = fmaxf(tm, __shfl_xor(tm, 32, IA_WAVE));
  const float m_new = fmaxf(c.m, tm);
  const float ref = (m_new == -INFINITY) ? 0.f : m_new;              // a column that has seen nothing yet
  const float corr = (c.m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(c.m - ref);
  float p[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) p[r] = ok[r] ? __builtin_amdgcn_exp2f(x[r] - ref) : 0.f;
  const f32x2_t w0 = {p[0], p[1]}, w1 = {p[2], p[3]};
  const uint32_t p0 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w0, bf16x2_t));
  const uint32_t p1 = __builtin_bit_cast(uint32_t, __builtin_convertvector(w1, bf16x2_t));
  const float sum = (bf16_bits_to_float((uint16_t)(p0 & 0xffffu)) + bf16_bits_to_float((uint16_t)(p0 >> 16))) +
                    (bf16_bits_to_float((uint16_t)(p1 & 0xffffu)) + bf16_bits_to_float((uint16_t)(p1 >> 16)));
  // most tiles leave every column's maximum where it was: the accumulators are rescaled only when one has moved
  if (__any(m_new != c.m)) {
    c.l *= corr;
#pragma unroll
    for (int n = 0; n < NSV; ++n) o[n] *= corr;
  }
  c.l += sum;
  c.m = m_new;
  return wp_s16x4(p0, p1);
}

// One tile of 16 keys, t0 .. t0 + 15, against the wave's 16 columns, in two halves so that the loads of the next tile
// fly while this one is worked on.  klo .. kmax: the keys that any column of the wave sees (the same in all lanes).
struct WpKeys {
  s16x4 kr[NSK];                 // this lane's key row
  uint2 v[NSV];                  // four keys' values of NSV channels
  uint32_t mlo, mhi;             // which of the four are keys that some column sees
};

template <bool POW2>
__device__ __forceinline__ void wp_load_keys(const WpGeom& G, int t0, int j, int qd, int klo, int kmax, WpKeys& T,
                                             bool& bad) {
  const int key = t0 + j;
  const int keyc = key > kmax ? kmax : (key < klo ? klo : key);
  const int page = G.bt[POW2 ? keyc >> G.ps_shift : keyc / G.ps];
  const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
  wp_load_row(G.k_base + (size_t)(page_ok ? page : 0) * G.k_page + (size_t)(POW2 ? keyc & (G.ps - 1) : keyc % G.ps) * WP_DIM,
              qd, T.kr);
  const int kg = t0 + 4 * qd;    // this lane brings the values of the keys kg .. kg + 3 (one quad, one page)
  const int kgc = kg > kmax ? (kmax & ~3) : (kg + 3 < klo ? (klo & ~3) : kg);
  const int pagev = G.bt[POW2 ? kgc >> G.ps_shift : kgc / G.ps];
  const bool pagev_ok = (unsigned)pagev < (unsigned)G.num_pages;
  const uint16_t* vq = G.v_base + (size_t)(pagev_ok ? pagev : 0) * G.v_page + (POW2 ? kgc & (G.ps - 1) : kgc % G.ps);
#pragma unroll
  for (int n = 0; n < NSV; ++n) T.v[n] = *reinterpret_cast<const uint2*>(vq + (size_t)(n * 16 + j) * G.ps);
  T.mlo = T.mhi = 0u;
  if (kg == kgc && pagev_ok) {
    T.mlo = ((kg >= klo && kg <= kmax) ? 0x0000ffffu : 0u) | ((kg + 1 >= klo && kg + 1 <= kmax) ? 0xffff0000u : 0u);
    T.mhi = ((kg + 2 >= klo && kg + 2 <= kmax) ? 0x0000ffffu : 0u) | ((kg + 3 >= klo && kg + 3 <= kmax) ? 0xffff0000u : 0u);
  }
  bad = bad || (key >= klo && key <= kmax && !page_ok) || (kg + 3 >= klo && kg <= kmax && !pagev_ok);
}

// This lane's column sees the keys lo .. pos (pos below zero: no such column).
__device__ __forceinline__ void wp_use_keys(const WpKeys& T, int t0, int qd, int lo, int pos, float scale_log2,
                                            const s16x4 (&q)[NSK], WpCol& c, f32x4 (&o)[NSV]) {
  const int kg = t0 + 4 * qd;
  f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < NSK; ++st) s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(T.kr[st], q[st], s, 0, 0, 0);
  bool ok[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) ok[r] = kg + r <= pos && kg + r >= lo;
  const s16x4 pw = wp_softmax_step(s, ok, scale_log2, c, o);
#pragma unroll
  for (int n = 0; n < NSV; ++n)
    o[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wp_s16x4(T.v[n].x & T.mlo, T.v[n].y & T.mhi), pw, o[n], 0, 0, 0);
}

// A tile without look ahead, in the halves of its loads: the keys, then (wp_work_tile) the values, both asked for before
// the first product.  Asking for the next tile's keys a tile ahead was measured too: 17 registers more, still three
// waves a SIMD, and 8% slower.  ``inner``: every column of the wave sees the tile whole and it lies in one page (pages of a multiple of 16 positions): the page is looked up
// once for the wave, the addresses are the wave's plus a lane's place, and neither scores, weights nor values need a
// mask.  Most tiles of a window are such tiles.
template <bool POW2>
__device__ __forceinline__ void wp_load_k(const WpGeom& G, int t0, int j, int qd, int klo, int kmax, bool inner,
                                          s16x4 (&kr)[NSK], bool& bad) {
  if (inner) {
    const int page = G.bt[POW2 ? t0 >> G.ps_shift : t0 / G.ps];
    const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
    bad = bad || !page_ok;
    const int off = POW2 ? t0 & (G.ps - 1) : t0 % G.ps;
    wp_load_row(G.k_base + (size_t)(page_ok ? page : 0) * G.k_page + (size_t)off * WP_DIM + j * WP_DIM, qd, kr);
    return;
  }
  const int key = t0 + j;
  const int keyc = key > kmax ? kmax : (key < klo ? klo : key);
  const int page = G.bt[POW2 ? keyc >> G.ps_shift : keyc / G.ps];
  const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
  wp_load_row(G.k_base + (size_t)(page_ok ? page : 0) * G.k_page + (size_t)(POW2 ? keyc & (G.ps - 1) : keyc % G.ps) * WP_DIM,
              qd, kr);
  bad = bad || (key >= klo && key <= kmax && !page_ok);
}

template <bool POW2>
__device__ __forceinline__ void wp_load_v(const WpGeom& G, int t0, int j, int qd, int klo, int kmax, bool inner,
                                          uint2 (&v)[NSV], uint32_t& mlo, uint32_t& mhi, bool& bad) {
  if (inner) {
    const int page = G.bt[POW2 ? t0 >> G.ps_shift : t0 / G.ps];
    const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
    bad = bad || !page_ok;
    const int off = POW2 ? t0 & (G.ps - 1) : t0 % G.ps;
    const uint16_t* vq = G.v_base + (size_t)(page_ok ? page : 0) * G.v_page + off + (size_t)j * G.ps + 4 * qd;
#pragma unroll
    for (int n = 0; n < NSV; ++n) v[n] = *reinterpret_cast<const uint2*>(vq + (size_t)n * 16 * G.ps);
    mlo = mhi = 0xffffffffu;
    return;
  }
  const int kg = t0 + 4 * qd;    // this lane brings the values of the keys kg .. kg + 3 (one quad, one page)
  const int kgc = kg > kmax ? (kmax & ~3) : (kg + 3 < klo ? (klo & ~3) : kg);
  const int pagev = G.bt[POW2 ? kgc >> G.ps_shift : kgc / G.ps];
  const bool pagev_ok = (unsigned)pagev < (unsigned)G.num_pages;
  const uint16_t* vq = G.v_base + (size_t)(pagev_ok ? pagev : 0) * G.v_page + (POW2 ? kgc & (G.ps - 1) : kgc % G.ps);
#pragma unroll
  for (int n = 0; n < NSV; ++n) v[n] = *reinterpret_cast<const uint2*>(vq + (size_t)(n * 16 + j) * G.ps);
  mlo = mhi = 0u;
  if (kg == kgc && pagev_ok) {
    mlo = ((kg >= klo && kg <= kmax) ? 0x0000ffffu : 0u) | ((kg + 1 >= klo && kg + 1 <= kmax) ? 0xffff0000u : 0u);
    mhi = ((kg + 2 >= klo && kg + 2 <= kmax) ? 0x0000ffffu : 0u) | ((kg + 3 >= klo && kg + 3 <= kmax) ? 0xffff0000u : 0u);
  }
  bad = bad || (kg + 3 >= klo && kg <= kmax && !pagev_ok);
}

// The work on a tile whose keys are in ``kr``; its values are asked for first and used last.
template <bool POW2>
__device__ __forceinline__ void wp_work_tile(const WpGeom& G, int t0, int j, int qd, int lo, int pos, int klo, int kmax,
                                             bool inner, float scale_log2, const s16x4 (&kr)[NSK], const s16x4 (&q)[NSK],
                                             WpCol& c, f32x4 (&o)[NSV], bool& bad) {
  uint2 v[NSV];
  uint32_t mlo, mhi;
  wp_load_v<POW2>(G, t0, j, qd, klo, kmax, inner, v, mlo, mhi, bad);
  f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < NSK; ++st) s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kr[st], q[st], s, 0, 0, 0);
  const int kg = t0 + 4 * qd;
  bool ok[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) ok[r] = inner || (kg + r <= pos && kg + r >= lo);
  const s16x4 pw = wp_softmax_step(s, ok, scale_log2, c, o);
#pragma unroll
  for (int n = 0; n < NSV; ++n)
    o[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wp_s16x4(v[n].x & mlo, v[n].y & mhi), pw, o[n], 0, 0, 0);
}

// The tiles first, first + step, ... up to the one that holds key kmax, each tile's loads asked for a tile ahead.
// CT: query heads of one key/value head that the wave takes for its rows; a tile that was loaded serves them all.
// AHEAD false: no tile is asked for ahead.
template <bool POW2, int CT, bool AHEAD>
__device__ __forceinline__ void wp_walk_keys(const WpGeom& G, int first, int step, int j, int qd, int lo, int pos, int klo,
                                             int kmax, float scale_log2, const s16x4 (&q)[CT][NSK], WpCol (&c)[CT],
                                             f32x4 (&o)[CT][NSV], bool& bad, int inner_lo = 0x7fffffff, int inner_hi = -1) {
  if (first > kmax) return;
  if (!AHEAD) {                  // a tile's loads and its work in turn: fewer registers, so more waves share a SIMD
    // inner_lo .. inner_hi: the keys that every column sees (tiles inside them take the short way)
    const bool whole_pages = (G.ps & 15) == 0;
    for (int t0 = first; t0 <= kmax; t0 += step) {
      const bool inner = whole_pages && t0 >= inner_lo && t0 + 15 <= inner_hi;
      s16x4 kr[NSK];
      wp_load_k<POW2>(G, t0, j, qd, klo, kmax, inner, kr, bad);
#pragma unroll
      for (int u = 0; u < CT; ++u)
        wp_work_tile<POW2>(G, t0, j, qd, lo, pos, klo, kmax, inner, scale_log2, kr, q[u], c[u], o[u], bad);
    }
    return;
  }
  WpKeys A, B;
  wp_load_keys<POW2>(G, first, j, qd, klo, kmax, A, bad);
  for (int t0 = first; t0 <= kmax; t0 += 2 * step) {
    const bool more = t0 + step <= kmax;
    if (more) wp_load_keys<POW2>(G, t0 + step, j, qd, klo, kmax, B, bad);
#pragma unroll
    for (int u = 0; u < CT; ++u) wp_use_keys(A, t0, qd, lo, pos, scale_log2, q[u], c[u], o[u]);
    if (!more) break;
    if (t0 + 2 * step <= kmax) wp_load_keys<POW2>(G, t0 + 2 * step, j, qd, klo, kmax, A, bad);
#pragma unroll
    for (int u = 0; u < CT; ++u) wp_use_keys(B, t0 + step, qd, lo, pos, scale_log2, q[u], c[u], o[u]);
  }
}

// One tile of 16 blocks, b0 .. b0 + 15.  This lane's column sees the blocks below nb; nbmax: the most any column sees.
template <bool POW2>
__device__ __forceinline__ void wp_tile_blocks(const WpGeom& G, int b0, int j, int qd, int nb, int nbmax,
                                               float scale_log2, const s16x4 (&q)[NSK], WpCol& c, f32x4 (&o)[NSV],
                                               bool& bad) {
  const int b = b0 + j < nbmax ? b0 + j : nbmax - 1;
  const int t = b * G.P + G.P - 1;
  const int page = G.btp[POW2 ? t >> G.ps_shift : t / G.ps];
  const bool page_ok = (unsigned)page < (unsigned)G.num_pool_pages;
  s16x4 kr[NSK];
  wp_load_row(G.pk_base + (size_t)(page_ok ? page : 0) * G.pk_page + (size_t)((POW2 ? t & (G.ps - 1) : t % G.ps) / G.P) * WP_DIM,
              qd, kr);
  bad = bad || (b0 + j < nbmax && !page_ok);
  f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < NSK; ++st) s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(kr[st], q[st], s, 0, 0, 0);
  bool ok[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) ok[r] = b0 + 4 * qd + r < nb;
  const s16x4 pw = wp_softmax_step(s, ok, scale_log2, c, o);
  // the values of the blocks b0 + 4 qd .. + 3, channel by channel, fetched after the scores are done with their
  // registers (blocks are few; what counts is that this path needs no more registers than the keys')
  const uint16_t* vr[4];
  bool have[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int bb = b0 + 4 * qd + r;
    const bool in = bb < nbmax;
    const int tt = (in ? bb : nbmax - 1) * G.P + G.P - 1;
    const int pg = G.btp[POW2 ? tt >> G.ps_shift : tt / G.ps];
    const bool pg_ok = (unsigned)pg < (unsigned)G.num_pool_pages;
    bad = bad || (in && !pg_ok);
    have[r] = in && pg_ok;
    vr[r] = G.pv_base + (size_t)(pg_ok ? pg : 0) * G.pv_page + (size_t)((POW2 ? tt & (G.ps - 1) : tt % G.ps) / G.P) * WP_VDIM + j;
  }
#pragma unroll
  for (int n = 0; n < NSV; ++n) {
    uint32_t x[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) x[r] = have[r] ? (uint32_t)vr[r][n * 16] : 0u;
    o[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wp_s16x4(x[0] | (x[1] << 16), x[2] | (x[3] << 16)), pw, o[n], 0, 0, 0);
  }
}

__device__ __forceinline__ WpGeom wp_geom(const uint16_t* k_pages, const uint16_t* v_pages, const uint16_t* pk_pages,
                                          const uint16_t* pv_pages, const int* bt_tok, int bt_tok_stride,
                                          const int* bt_pool, int bt_pool_stride, int row, int g, int nkv, int ps,
                                          int num_pages, int num_pool_pages, int P) {
  WpGeom G;
  G.k_page = (size_t)nkv * ps * WP_DIM;
  G.v_page = (size_t)nkv * ps * WP_VDIM;
  G.k_base = k_pages + (size_t)g * ps * WP_DIM;
  G.v_base = v_pages + (size_t)g * ps * WP_VDIM;
  G.bt = bt_tok + (size_t)row * bt_tok_stride;
  G.ps = ps;
  G.ps_shift = 31 - __clz(ps);
  G.num_pages = num_pages;
  G.P = P > 0 ? P : 1;
  G.E = (ps - 1) / G.P + 1;
  G.pk_page = (size_t)nkv * G.E * WP_DIM;
  G.pv_page = (size_t)nkv * G.E * WP_VDIM;
  G.pk_base = pk_pages ? pk_pages + (size_t)g * G.E * WP_DIM : nullptr;
  G.pv_base = pv_pages ? pv_pages + (size_t)g * G.E * WP_VDIM : nullptr;
  G.btp = bt_pool ? bt_pool + (size_t)row * bt_pool_stride : nullptr;
  G.num_pool_pages = num_pool_pages;
  return G;
}

__device__ __forceinline__ int wp_first_key(int pos, int window) { return window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0; }
__device__ __forceinline__ int wp_blocks_seen(int pos, int window, int P) {
  return (window > 0 && P > 0 && pos - window + 1 >= P) ? (pos - window + 1) / P : 0;
}

__device__ __forceinline__ void wp_store_bf16x4(uint16_t* at, const f32x4& x, float f) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(x[0] * f) | ((uint32_t)float_to_bf16_bits(x[1] * f) << 16);
  u.y = (uint32_t)float_to_bf16_bits(x[2] * f) | ((uint32_t)float_to_bf16_bits(x[3] * f) << 16);
  *reinterpret_cast<uint2*>(at) = u;
}

// ------------------------------------------------------------------------ portions of prompts
// 256 threads; a workgroup takes 16 consecutive rows of one query head (a quarter of a tile (request, first row) of 64
// rows that the host lists): the 16 columns are those rows, and the tiles of blocks and of keys are dealt out over the
// four waves, which join through LDS in the order of the waves, as for single tokens.  A wave alone on 16 rows would
// walk up to window / 16 tiles one after the other, each a chain of dependent matrix instructions, exchanges and
// exponentials, with two such waves a SIMD at 2,048 rows and 16 heads: the rows' keys in four parts make four times
// the waves, and without a tile asked for ahead the kernel's registers let three of them share a SIMD (at head sizes
// of 128: 139 registers; held to the 128 of four waves, a dozen values went to scratch and nothing was gained).
// Workgroups are numbered so that the heads of one tile follow each other.
template <bool POW2>
__global__ __launch_bounds__(256) void wpa_prefill_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const uint16_t* __restrict__ pk_pages, const uint16_t* __restrict__ pv_pages,
    uint16_t* __restrict__ out, const float* __restrict__ sinks, const int* __restrict__ seq_starts,
    const int* __restrict__ seq_ctx, const int* __restrict__ bt_tok, int bt_tok_stride, const int* __restrict__ bt_pool,
    int bt_pool_stride, const int* __restrict__ tiles, int nh, int nkv, int ps, int num_pages, int num_pool_pages,
    float scale_log2, int window, int P) {
  __shared__ f32x4 red[3][NSV][64];
  __shared__ float s_m[4][16], s_l[4][64];
  __shared__ int s_bad;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, qd = lane >> 4;
  const int lin = blockIdx.x;
  const int tile = lin / (4 * nh), rest = lin - tile * 4 * nh;
  const int sub = rest / nh, h = rest - sub * nh;
  const int sidx = tiles[2 * tile], row0 = tiles[2 * tile + 1];
  const int qstart = seq_starts[sidx], qlen = seq_starts[sidx + 1] - qstart, ctx = seq_ctx[sidx];
  const int rb = row0 + sub * 16;
  if (rb >= qlen) return;                                   // the whole workgroup: no barrier has been met
  if (tid == 0) s_bad = 0;
  const int g = h / (nh / nkv);
  const int row = rb + j;
  const bool col_ok = row < qlen;
  const int pos = col_ok ? ctx + row : -1;
  const int kmax = ctx + (rb + 15 < qlen ? rb + 15 : qlen - 1);
  const int klo = wp_first_key(ctx + rb, window);
  const int lo = wp_first_key(pos, window);
  const int nb = col_ok ? wp_blocks_seen(pos, window, P) : 0, nbmax = wp_blocks_seen(kmax, window, P);
  const WpGeom G = wp_geom(k_pages, v_pages, pk_pages, pv_pages, bt_tok, bt_tok_stride, bt_pool, bt_pool_stride, sidx, g,
                           nkv, ps, num_pages, num_pool_pages, P);
  const size_t qrow = (size_t)(qstart + (col_ok ? row : rb));
  s16x4 qr1[1][NSK];
  s16x4 (&qr)[NSK] = qr1[0];
  wp_load_row(q + qrow * q_stride + (size_t)h * WP_DIM, qd, qr);
  f32x4 o1[1][NSV];
  f32x4 (&o)[NSV] = o1[0];
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  WpCol c1[1];
  WpCol& c = c1[0];
  c.m = -INFINITY;
  c.l = 0.f;
  bool bad = false;
  const int block_tiles = (nbmax + 15) / 16;
  for (int i = wave; i < block_tiles; i += 4) wp_tile_blocks<POW2>(G, i * 16, j, qd, nb, nbmax, scale_log2, qr, c, o, bad);
  const int turn = (wave + 4 - block_tiles % 4) % 4;
  // every column sees the keys from the last row's first key to the first row's own (when all 16 rows are there)
  const bool all_rows = rb + 15 < qlen;
  wp_walk_keys<POW2, 1, false>(G, (klo / 16 + turn) * 16, 64, j, qd, lo, pos, klo, kmax, scale_log2, qr1, c1, o1, bad,
                               all_rows ? wp_first_key(kmax, window) : 0x7fffffff, all_rows ? ctx + rb : -1);
  // ---- the waves meet: a common maximum, then sums in the order of the waves
  if (qd == 0) s_m[wave][j] = c.m;
  __syncthreads();
  if (bad) s_bad = 1;
  const float M = fmaxf(fmaxf(s_m[0][j], s_m[1][j]), fmaxf(s_m[2][j], s_m[3][j]));
  const float f = (c.m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(c.m - M);
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] *= f;
  s_l[wave][lane] = c.l * f;
  if (wave > 0) {
#pragma unroll
    for (int n = 0; n < NSV; ++n) red[wave - 1][n][lane] = o[n];
  }
  __syncthreads();
  if (wave > 0 || !col_ok) return;
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = ((o[n] + red[0][n][lane]) + red[1][n][lane]) + red[2][n][lane];
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w)
#pragma unroll
    for (int x = 0; x < 4; ++x) l += s_l[w][x * 16 + j];
  if (sinks) l += __builtin_amdgcn_exp2f(sinks[h] * WP_LOG2E - M);
  float inv = 1.0f / l;
  if (s_bad) inv = __uint_as_float(0x7fc00000u);
  uint16_t* at = out + (qrow * nh + h) * WP_VDIM + 4 * qd;
#pragma unroll
  for (int n = 0; n < NSV; ++n) wp_store_bf16x4(at + n * 16, o[n], inv);
}

// ------------------------------------------------------------------------ single tokens
// grid (B, nkv * ceil(G / 16)), 256 threads.  Token b is row b of q and out and of the block tables.
template <bool POW2>
__global__ __launch_bounds__(256) void wpa_decode_kernel(
    const uint16_t* __restrict__ q, int q_stride, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const uint16_t* __restrict__ pk_pages, const uint16_t* __restrict__ pv_pages,
    uint16_t* __restrict__ out, const float* __restrict__ sinks, const int* __restrict__ positions,
    const int* __restrict__ bt_tok, int bt_tok_stride, const int* __restrict__ bt_pool, int bt_pool_stride, int nh,
    int nkv, int ps, int num_pages, int num_pool_pages, float scale_log2, int window, int P) {
  __shared__ f32x4 red[3][NSV][64];
  __shared__ float s_m[4][16], s_l[4][64];
  __shared__ int s_bad;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, j = lane & 15, qd = lane >> 4;
  const int b = blockIdx.x;
  const int Gq = nh / nkv, HC = (Gq + 15) / 16;
  const int g = blockIdx.y / HC, hc = blockIdx.y - g * HC;
  const int hj = hc * 16 + j;
  const bool col_ok = hj < Gq;
  const int h = g * Gq + (col_ok ? hj : 0);
  const int p = positions[b];
  if (tid == 0) s_bad = 0;
  const WpGeom G = wp_geom(k_pages, v_pages, pk_pages, pv_pages, bt_tok, bt_tok_stride, bt_pool, bt_pool_stride, b, g, nkv,
                           ps, num_pages, num_pool_pages, P);
  s16x4 qr1[1][NSK];
  s16x4 (&qr)[NSK] = qr1[0];
  wp_load_row(q + (size_t)b * q_stride + (size_t)h * WP_DIM, qd, qr);
  f32x4 o1[1][NSV];
  f32x4 (&o)[NSV] = o1[0];
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  WpCol c1[1];
  WpCol& c = c1[0];
  c.m = -INFINITY;
  c.l = 0.f;
  bool bad = false;
  const int lo = wp_first_key(p, window), nb = wp_blocks_seen(p, window, P);
  const int pos = col_ok ? p : -1, nbc = col_ok ? nb : 0;
  const int block_tiles = (nb + 15) / 16;
  for (int i = wave; i < block_tiles; i += 4) wp_tile_blocks<POW2>(G, i * 16, j, qd, nbc, nb, scale_log2, qr, c, o, bad);
  // the tiles of keys go round the waves from where the tiles of blocks stopped, so that no wave has two more
  const int turn = (wave + 4 - block_tiles % 4) % 4;
  wp_walk_keys<POW2, 1, true>(G, (lo / 16 + turn) * 16, 64, j, qd, lo, pos, lo, p, scale_log2, qr1, c1, o1, bad);
  // ---- the waves meet: a common maximum, then sums in the order of the waves
  if (qd == 0) s_m[wave][j] = c.m;
  __syncthreads();
  if (bad) s_bad = 1;
  float M = fmaxf(fmaxf(s_m[0][j], s_m[1][j]), fmaxf(s_m[2][j], s_m[3][j]));
  const float f = (c.m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(c.m - M);
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] *= f;
  s_l[wave][lane] = c.l * f;
  if (wave > 0) {
#pragma unroll
    for (int n = 0; n < NSV; ++n) red[wave - 1][n][lane] = o[n];
  }
  __syncthreads();
  if (wave > 0 || !col_ok) return;
#pragma unroll
  for (int n = 0; n < NSV; ++n) o[n] = ((o[n] + red[0][n][lane]) + red[1][n][lane]) + red[2][n][lane];
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w)
#pragma unroll
    for (int x = 0; x < 4; ++x) l += s_l[w][x * 16 + j];
  if (sinks) l += __builtin_amdgcn_exp2f(sinks[h] * WP_LOG2E - M);
  float inv = 1.0f / l;
  if (s_bad) inv = __uint_as_float(0x7fc00000u);
  uint16_t* at = out + ((size_t)b * nh + h) * WP_VDIM + 4 * qd;
#pragma unroll
  for (int n = 0; n < NSV; ++n) wp_store_bf16x4(at + n * 16, o[n], inv);
}

// ------------------------------------------------------------------------ launchers
extern "C" int ia_wpa_mfma_dim() { return WP_DIM; }
extern "C" int ia_wpa_mfma_vdim() { return WP_VDIM; }

static int wp_check(int nh, int nkv, int ps, int num_pages, int bt_stride, int q_stride, int window, int P,
                    const void* pk, const void* pv, const int* bt_pool, int bt_pool_stride, int num_pool_pages) {
  if (nh <= 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || (ps & 3) || num_pages <= 0 || bt_stride <= 0 ||
      q_stride < nh * WP_DIM || window < 0 || P < 0)
    return IA_ERR_BAD_ARG;
  if (window > 0 && P > 0 && (!pk || !pv || !bt_pool || bt_pool_stride <= 0 || num_pool_pages <= 0)) return IA_ERR_BAD_ARG;
  if (q_stride & 7) return IA_ERR_UNSUPPORTED;              // 16-byte loads of the queries
  return IA_OK;
}

// q rows of q_stride bf16 values (head h's WP_DIM values from h WP_DIM); out [N, nh WP_VDIM] bf16; tiles[i] =
// (request, first row of a tile of 64 among the request's rows); request s has the rows seq_starts[s] ..
// seq_starts[s + 1] - 1 of q and out, seq_ctx[s] keys before its first row, and row s of both block tables.
extern "C" int ia_wpa_prefill(const void* q, int q_stride, const void* k_pages, const void* v_pages, const void* pk_pages,
                              const void* pv_pages, void* out, const float* sinks, const int* seq_starts,
                              const int* seq_ctx, const int* bt_tok, int bt_tok_stride, const int* bt_pool,
                              int bt_pool_stride, const int* tiles, int num_tiles, int nh, int nkv, int ps,
                              int num_pages, int num_pool_pages, float scale, int window, int P, hipStream_t stream) {
  if (num_tiles < 0) return IA_ERR_BAD_ARG;
  const int rc = wp_check(nh, nkv, ps, num_pages, bt_tok_stride, q_stride, window, P, pk_pages, pv_pages, bt_pool,
                          bt_pool_stride, num_pool_pages);
  if (rc != IA_OK) return rc;
  if (num_tiles == 0) return IA_OK;
  if (!q || !k_pages || !v_pages || !out || !tiles || !seq_starts || !seq_ctx || !bt_tok) return IA_ERR_BAD_ARG;
  if ((long long)num_tiles * nh > 0x7fffffffLL) return IA_ERR_UNSUPPORTED;
  if (!(window > 0 && P > 0)) P = 0;
  if ((long long)num_tiles * nh * 4 > 0x7fffffffLL) return IA_ERR_UNSUPPORTED;
#define WP_PRE(P2)                                                                                                 \
  wpa_prefill_kernel<P2><<<num_tiles * nh * 4, 256, 0, stream>>>(                                                  \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, (const uint16_t*)pk_pages, \
      (const uint16_t*)pv_pages, (uint16_t*)out, sinks, seq_starts, seq_ctx, bt_tok, bt_tok_stride, bt_pool,       \
      bt_pool_stride, tiles, nh, nkv, ps, num_pages, num_pool_pages, scale * WP_LOG2E, window, P)
  if ((ps & (ps - 1)) == 0) WP_PRE(true);
  else WP_PRE(false);
#undef WP_PRE
  IA_LAUNCH_CHECK();
  return IA_OK;
}

extern "C" int ia_wpa_decode(const void* q, int q_stride, const void* k_pages, const void* v_pages, const void* pk_pages,
                             const void* pv_pages, void* out, const float* sinks, const int* positions, const int* bt_tok,
                             int bt_tok_stride, const int* bt_pool, int bt_pool_stride, int B, int nh, int nkv, int ps,
                             int num_pages, int num_pool_pages, float scale, int window, int P, hipStream_t stream) {
  if (B < 0) return IA_ERR_BAD_ARG;
  const int rc = wp_check(nh, nkv, ps, num_pages, bt_tok_stride, q_stride, window, P, pk_pages, pv_pages, bt_pool,
                          bt_pool_stride, num_pool_pages);
  if (rc != IA_OK) return rc;
  if (B == 0) return IA_OK;
  if (!q || !k_pages || !v_pages || !out || !positions || !bt_tok) return IA_ERR_BAD_ARG;
  const int HC = (nh / nkv + 15) / 16;
  if ((long long)nkv * HC > 65535) return IA_ERR_UNSUPPORTED;
  if (!(window > 0 && P > 0)) P = 0;
  dim3 grid(B, nkv * HC);
#define WP_DEC(P2)                                                                                                 \
  wpa_decode_kernel<P2><<<grid, 256, 0, stream>>>(                                                                 \
      (const uint16_t*)q, q_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, (const uint16_t*)pk_pages, \
      (const uint16_t*)pv_pages, (uint16_t*)out, sinks, positions, bt_tok, bt_tok_stride, bt_pool, bt_pool_stride, \
      nh, nkv, ps, num_pages, num_pool_pages, scale * WP_LOG2E, window, P)
  if ((ps & (ps - 1)) == 0) WP_DEC(true);
  else WP_DEC(false);
#undef WP_DEC
  IA_LAUNCH_CHECK();
  return IA_OK;
}

#include "op_call.h"
IA_OP(ia_wpa_prefill)
IA_OP(ia_wpa_decode)
