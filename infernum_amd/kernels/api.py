"""Python face of the HIP kernels: shape checks on the host, then one C call.

Every function checks that its operands are what the kernel and its grid assume
(device, dtype, contiguity, sizes) before anything is launched, and launches on
torch's current stream, so that calls order with torch's own work and can be
captured into a HIP graph.  There is no fallback: without a GPU or without the
built library a call raises :class:`KernelError`.
"""
from __future__ import annotations

import atexit
import ctypes
import functools
import math
import os
import sys
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..csrc import build as _build


class KernelError(RuntimeError):
    pass


class KernelUnsupported(KernelError):
    """The kernel (or the library) does not take this size; nothing was launched."""


DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
GENERIC_MAX_HEAD_DIM = 640         # the plain attention kernel's limit (AG_MAX_D)
_libs: Dict[str, ctypes.CDLL] = {}

_ERRORS = {10001: "bad argument", 10002: "size not supported by this kernel",
           10003: "a call into the GEMM library failed"}


# Into how many parts the weight-streaming product splits the inner dimension of a weight [N, K], where that was
# measured and differs from the rule of sizes (about 512 workgroups): the 13B, 70B and 1B shapes' products on an
# MI355X, with cold weights and the norm that joins the parts behind them, at 1, 8 and 64 rows (13B down projection:
# 35.0 us in six even parts of nine chunks, 42.3 in the rule's seven; 70B QKV: 35.4 us in three parts, 43.5 in four).
# The sums of a product are taken in the order that its number of parts gives: a shape's entry is part of its
# arithmetic, the same in every process.
KNOWN_SPLITS = {
    (15360, 5120): 2, (5120, 5120): 5, (5120, 13824): 6,       # Llama-2-13B: QKV, output and down projection
    (10240, 8192): 3,                                          # Llama-3.1-70B: QKV
    (2048, 8192): 8,                                           # Llama-3.2-1B: down projection
}


def load_library(name: str) -> ctypes.CDLL:
    lib = _libs.get(name)
    if lib is None:
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: infernum_amd runs on a gfx950 GPU only (there is no CPU fallback)")
        try:
            path = _build.ensure(name)
            lib = ctypes.CDLL(path)
        except (OSError, _build.BuildError) as e:
            raise KernelError(f"the HIP kernel library '{name}' could not be built or loaded: {e}") from e
        if name == "core":
            for (N, K), parts in KNOWN_SPLITS.items():
                _ok(lib.ia_gemm_skinny_set_splits(N, K, parts), "gemm_skinny_set_splits")
        _libs[name] = lib
    return lib


def _core() -> ctypes.CDLL:
    return load_library("core")


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_fixed_stream: Optional[ctypes.c_void_p] = None


def _stream() -> ctypes.c_void_p:
    if _fixed_stream is not None:
        return _fixed_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class on_current_stream:
    """Within this block every kernel call launches on the stream that is current at its entry, looked up
    once (the lookup costs as much as several launches).  Enter it anew inside a graph capture: the capture
    has a stream of its own."""

    def __enter__(self):
        global _fixed_stream
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: infernum_amd runs on a gfx950 GPU only (there is no CPU fallback)")
        self._before = _fixed_stream
        _fixed_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _fixed_stream
        _fixed_stream = self._before
        return False


def _ok(code: int, what: str) -> None:
    if code != 0:
        why = _ERRORS.get(code, f"HIP error {code}")
        raise (KernelUnsupported if code == 10002 else KernelError)(f"{what}: {why}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "operand is not on the GPU")
            _need(t.is_contiguous(), "operand is not contiguous")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    _need(t.dtype == torch.int32 and t.is_cuda and t.is_contiguous() and t.numel() >= n,
          f"{what}: needs a contiguous int32 GPU tensor of at least {n} elements")


# --------------------------------------------------------------------------- rows
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[n, :] = float(table[ids[n], :]) * scale; out is fp32 [N, H]."""
    _dev(table, ids, out)
    V, H = table.shape
    N = ids.numel()
    _need(table.dtype in DTYPE_CODE, f"embed: table dtype {table.dtype}")
    _i32(ids, N, "embed ids")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (N, H), f"embed: out must be fp32 [{N}, {H}]")
    _ok(_core().ia_embed(_p(table), DTYPE_CODE[table.dtype], _p(ids), _p(out), N, H, V, ctypes.c_float(scale),
                         _stream()), "embed")
    return out


class SplitSum:
    """A matrix [M, N] given as a stack of fp32 partial sums ``parts`` [S, M, N]: what a matrix product
    whose inner dimension was split over workgroups leaves.  The kernels that take the product next
    (residual add + norm, rotary + cache write) add the parts themselves, in the order of their index."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor):
        if parts.dim() != 3 or parts.dtype != torch.float32 or not parts.is_contiguous():
            raise KernelError("SplitSum: parts must be a contiguous fp32 [S, M, N] tensor")
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def joined(self, dtype: torch.dtype) -> torch.Tensor:
        """The sum as one tensor (a library reduction; for paths that are not hot)."""
        return self.parts.sum(dim=0).to(dtype)


def add_rmsnorm(h: torch.Tensor, delta, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h += delta (fp32, in place); out = h * rsqrt(mean(h^2) + eps) * weight.

    ``delta`` is None, a tensor of h's shape in out's dtype, or a :class:`SplitSum`.
    With ``rows`` the norm is taken of the selected rows only and h stays as it is.
    """
    split = isinstance(delta, SplitSum)
    d = delta.parts if split else delta
    _dev(h, d, weight, out, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2, "add_rmsnorm: h must be fp32 [N, H]")
    H = h.shape[1]
    n_out = rows.numel() if rows is not None else h.shape[0]
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (n_out, H), f"add_rmsnorm: out must be [{n_out}, {H}]")
    splits, d_rows, d_code = 1, h.shape[0], DTYPE_CODE[out.dtype]
    if split:
        _need(tuple(d.shape[1:]) == tuple(h.shape), "add_rmsnorm: partial sums must be [S, N, H]")
        splits, d_code = d.shape[0], DTYPE_CODE[torch.float32]
    elif d is not None:
        _need(d.dtype == out.dtype and tuple(d.shape) == tuple(h.shape),
              "add_rmsnorm: delta must have h's shape and out's dtype")
    _need(weight.dtype in DTYPE_CODE and weight.numel() == H, f"add_rmsnorm: weight must hold {H} values")
    if rows is not None:
        _i32(rows, n_out, "add_rmsnorm rows")
    _ok(_core().ia_add_rmsnorm(_p(h), _p(d), d_code, splits, d_rows, DTYPE_CODE[out.dtype], _p(weight),
                               DTYPE_CODE[weight.dtype], _p(out), _p(rows), n_out, H, ctypes.c_float(eps),
                               _stream()), "add_rmsnorm")
    return out


def norm_add(h: torch.Tensor, delta, weight: torch.Tensor, eps: float, x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h += delta * rsqrt(mean(delta^2) + eps) * weight (fp32, in place): the norm sits on the branch's output.

    ``delta`` is a tensor of h's shape in the activations' dtype or a :class:`SplitSum`.  ``x`` (optional,
    h's shape in the activations' dtype) receives the new h, rounded once: what the next sublayer reads."""
    split = isinstance(delta, SplitSum)
    d = delta.parts if split else delta
    _dev(h, d, weight, x)
    _need(h.dtype == torch.float32 and h.dim() == 2, "norm_add: h must be fp32 [N, H]")
    N, H = h.shape
    splits, d_rows = 1, N
    if split:
        _need(d.shape[1] >= N and d.shape[2] == H, "norm_add: partial sums must be [S, >= N, H]")
        splits, d_rows = d.shape[0], d.shape[1]
    else:
        _need(d is not None and d.dtype in DTYPE_CODE and tuple(d.shape) == (N, H), "norm_add: delta must have h's shape")
    _need(weight.dtype in DTYPE_CODE and weight.numel() == H, f"norm_add: weight must hold {H} values")
    act = x.dtype if x is not None else (torch.bfloat16 if d.dtype == torch.bfloat16 else torch.float32)
    if x is not None:
        _need(x.dtype in DTYPE_CODE and tuple(x.shape) == (N, H), "norm_add: x must have h's shape")
        _need(split or x.dtype == d.dtype, "norm_add: x must have delta's dtype")
    _ok(_core().ia_norm_add(_p(h), _p(d), DTYPE_CODE[d.dtype], splits, d_rows, _p(weight), DTYPE_CODE[weight.dtype],
                            _p(x), DTYPE_CODE[act], N, H, ctypes.c_float(eps), _stream()), "norm_add")
    return h


ACTIVATIONS = {"gelu_tanh": 1, "gelu": 2, "relu_squared": 3}


def activation(x: torch.Tensor, kind: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = act(x) element by element in fp32 (in place without ``out``).  Kinds: gelu_tanh, gelu (the erf form), relu_squared."""
    out = x if out is None else out
    _dev(x, out)
    _need(kind in ACTIVATIONS, f"activation: unknown kind {kind!r}; known: {sorted(ACTIVATIONS)}")
    _need(x.dtype in DTYPE_CODE and out.dtype == x.dtype and out.numel() == x.numel(), "activation: out like x")
    _ok(_core().ia_activation(_p(x), _p(out), DTYPE_CODE[x.dtype], ctypes.c_size_t(x.numel()), ACTIVATIONS[kind],
                              _stream()), "activation")
    return out


def latent_prepare(proj: torch.Tensor, out: torch.Tensor, norm_weight: torch.Tensor, eps: float, H: int, dn: int,
                   dr: int, rank: int, latent: Optional[torch.Tensor] = None, latent_col: int = 0) -> torch.Tensor:
    """From rows [H heads of (dn plain | dr rotated) query values | rank latent values | dr key values | ...]
    the rows [H heads of (dr | rank) | key (dr | rank) | value (dr | rank)] that the attention kernels take with
    one key/value head (``latent``: the rank latent values and dr key values stand in rows of their own, from column
    ``latent_col`` on, and ``proj`` holds the queries alone): the rotated query parts at the heads' fronts (the rank places of the query heads are
    left for :func:`gemm_heads`), key = (k_rot, c), value = (0, c), c = RMSNorm(latent) * norm_weight."""
    _dev(proj, out, norm_weight)
    N = proj.shape[0]
    _need(proj.dim() == 2 and out.dim() == 2 and out.shape[0] == N and proj.dtype == out.dtype
          and proj.dtype in DTYPE_CODE, "latent_prepare: two matrices of one dtype with the same rows")
    _need(proj.shape[1] >= H * (dn + dr) + (0 if latent is not None else rank + dr)
          and out.shape[1] >= (H + 2) * (dr + rank), "latent_prepare: rows too short for their heads")
    lat_ptr, lat_stride = None, 0
    if latent is not None:
        _dev(latent)
        _need(latent.dim() == 2 and latent.shape[0] == N and latent.dtype == proj.dtype and latent.stride(1) == 1
              and latent_col >= 0 and latent.shape[1] >= latent_col + rank + dr, "latent_prepare: the latent's rows")
        lat_ptr = ctypes.c_void_p(latent.data_ptr() + latent_col * latent.element_size())
        lat_stride = int(latent.stride(0))
    _need(norm_weight.dtype in DTYPE_CODE and norm_weight.numel() == rank, f"latent_prepare: {rank} norm weights")
    _ok(_core().ia_latent_prepare(_p(proj), proj.shape[1], lat_ptr, lat_stride, _p(out), out.shape[1], DTYPE_CODE[out.dtype],
                                  _p(norm_weight), DTYPE_CODE[norm_weight.dtype], N, H, dn, dr, rank,
                                  ctypes.c_float(eps), _stream()), "latent_prepare")
    return out


def gemm_heads(x: torch.Tensor, x_offset: int, x_head: int, w: torch.Tensor, out: torch.Tensor, out_offset: int,
               out_head: int, gate: Optional[torch.Tensor] = None, gate_offset: int = 0) -> torch.Tensor:
    """out[n, out_offset + h out_head + j] = sum_k x[n, x_offset + h x_head + k] w[h, j, k], for every head h of
    w [H, J, K]; with ``gate`` times sigmoid(gate[n, gate_offset + h J + j]).  x, out and gate are matrices of one
    dtype with the same rows; the offsets and head strides are in elements."""
    _dev(x, w, out, gate)
    _need(w.dim() == 3 and x.dim() == 2 and out.dim() == 2 and x.shape[0] == out.shape[0], "gemm_heads: shapes")
    H, J, Kd = w.shape
    N = x.shape[0]
    _need(x.dtype == w.dtype == out.dtype and x.dtype in DTYPE_CODE, "gemm_heads: one dtype")
    _need(x_offset >= 0 and x_offset + (H - 1) * x_head + Kd <= x.shape[1], "gemm_heads: x's rows are too short")
    _need(out_offset >= 0 and out_offset + (H - 1) * out_head + J <= out.shape[1], "gemm_heads: out's rows are too short")
    esz = x.element_size()
    gp, g_row = None, 0
    if gate is not None:
        _need(gate.dim() == 2 and gate.shape[0] == N and gate.dtype == x.dtype
              and gate_offset >= 0 and gate_offset + H * J <= gate.shape[1], "gemm_heads: gate")
        gp, g_row = ctypes.c_void_p(gate.data_ptr() + gate_offset * esz), gate.shape[1]
    _ok(_core().ia_gemm_heads(ctypes.c_void_p(x.data_ptr() + x_offset * esz), x.shape[1], x_head, _p(w),
                              ctypes.c_void_p(out.data_ptr() + out_offset * esz), out.shape[1], out_head,
                              gp, g_row, DTYPE_CODE[x.dtype], N, H, J, Kd, _stream()), "gemm_heads")
    return out


def router_topk(logits: torch.Tensor, bias: Optional[torch.Tensor], top: int):
    """-> (ids int32 [N, top], weights fp32 [N, top]): the ``top`` largest of logits + bias per row (the lowest
    index among equals) and the softmax over those alone."""
    _dev(logits, bias)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "router_topk: fp32 logits [N, E]")
    N, E = logits.shape
    _need(0 < top <= E, f"router_topk: top must be 1 .. {E}")
    _need(bias is None or (bias.dtype in DTYPE_CODE and bias.numel() == E), f"router_topk: {E} biases")
    ids = torch.empty((N, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((N, top), dtype=torch.float32, device=logits.device)
    _ok(_core().ia_router_topk(_p(logits), _p(bias), DTYPE_CODE[bias.dtype] if bias is not None else 0, _p(ids),
                               _p(weights), N, E, top, _stream()), "router_topk")
    return ids, weights


def gemm_mfma_grouped(x: torch.Tensor, w: torch.Tensor, rows_at: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[rows_at[g] : rows_at[g + 1]] = x[rows_at[g] : rows_at[g + 1]] @ w[g]^T for every group g: x [rows, K] and
    w [groups, N, K] in bf16, rows_at int32 [groups + 1] on the device, rising from 0 to at most rows (nothing of it
    is read on the host; rows past rows_at[-1] are left as they are).  K must be a multiple of 64."""
    _dev(x, w, rows_at, out)
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 3
          and w.shape[2] == x.shape[1], "gemm_mfma_grouped: x [rows, K] and w [groups, N, K] in bf16")
    G, N, Kd = w.shape
    _i32(rows_at, G + 1, "gemm_mfma_grouped rows_at")
    if out is None:
        out = torch.empty((x.shape[0], N), dtype=torch.bfloat16, device=x.device)
    _need(out.dtype == torch.bfloat16 and tuple(out.shape) == (x.shape[0], N), "gemm_mfma_grouped: out [rows, N] in bf16")
    _ok(_core().ia_gemm_mfma_grouped(_p(x), _p(w), _p(out), _p(rows_at), G, x.shape[0], N, Kd, _stream()),
        "gemm_mfma_grouped")
    return out


MOE_GROUPED_ROWS_AN_EXPERT = 48


def moe_grouped_from_tokens(E: int, top: int, W: int, ff: int, dtype: torch.dtype) -> int:
    """From how many tokens of a step on the routed experts take the grouped form of the LDS-tiled product (an
    expert then has some tens of rows on average); 0: never (32-bit, or sizes that product does not take: its
    inner dimensions W and ff must be multiples of 64)."""
    if dtype != torch.bfloat16 or W % 64 or ff % 64:
        return 0
    return -(-MOE_GROUPED_ROWS_AN_EXPERT * E // top)


def moe_grouped_rows(N: int, E: int, top: int, W: int, ff: int, dtype: torch.dtype) -> bool:
    first = moe_grouped_from_tokens(E, top, W, ff, dtype)
    return first > 0 and N >= first


def moe_experts(x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_gate_up: torch.Tensor,
                w_down: torch.Tensor, limit: float, alpha: float) -> SplitSum:
    """The chosen experts of every token: w_gate_up [E, 2 ff, W] with the gate's and up's rows alternating,
    w_down [E, W, ff].  y = g sigmoid(alpha g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit).
    Returns fp32 parts [top, N, W], each already times its routing weight."""
    _dev(x, ids, weights, w_gate_up, w_down)
    N, W = x.shape
    E, two_ff, _ = w_gate_up.shape
    ff = two_ff // 2
    top = ids.shape[1]
    _need(x.dtype in DTYPE_CODE and w_gate_up.dtype == x.dtype and w_down.dtype == x.dtype, "moe: one dtype")
    _need(tuple(w_gate_up.shape) == (E, 2 * ff, W) and tuple(w_down.shape) == (E, W, ff), "moe: weights' shapes")
    _need(ids.dtype == torch.int32 and tuple(ids.shape) == (N, top) and weights.dtype == torch.float32
          and tuple(weights.shape) == (N, top), "moe: ids int32 and weights fp32 [N, top]")
    P = N * top
    offsets = torch.empty(E + 1, dtype=torch.int32, device=x.device)
    perm = torch.empty(max(P, 1), dtype=torch.int32, device=x.device)
    y = torch.empty((max(P, 1), ff), dtype=x.dtype, device=x.device)
    parts = torch.empty((top, N, W), dtype=torch.float32, device=x.device)
    code = DTYPE_CODE[x.dtype]
    _ok(_core().ia_moe_sort(_p(ids), _p(offsets), _p(perm), P, E, _stream()), "moe_sort")
    if moe_grouped_rows(N, E, top, W, ff, x.dtype):
        # many rows an expert: the tokens' rows in the order of the sort, the LDS-tiled product expert by expert
        xs = torch.empty((P, W), dtype=x.dtype, device=x.device)
        gu = torch.empty((P, 2 * ff), dtype=x.dtype, device=x.device)
        _ok(_core().ia_moe_gather(_p(x), _p(perm), _p(xs), P, top, W, _stream()), "moe_gather")
        gemm_mfma_grouped(xs, w_gate_up, offsets, gu)
        _ok(_core().ia_moe_glu(_p(gu), _p(y), P, ff, ctypes.c_float(limit), ctypes.c_float(alpha), _stream()), "moe_glu")
        gemm_mfma_grouped(y, w_down, offsets, xs)
        _ok(_core().ia_moe_scatter(_p(xs), _p(perm), _p(weights), _p(parts), N, top, W, _stream()), "moe_scatter")
        return SplitSum(parts)
    _ok(_core().ia_moe_gate_up(_p(x), _p(w_gate_up), _p(y), _p(offsets), _p(perm), code, P, E, top, W, ff,
                               ctypes.c_float(limit), ctypes.c_float(alpha), _stream()), "moe_gate_up")
    _ok(_core().ia_moe_down(_p(y), _p(w_down), _p(parts), _p(weights), _p(offsets), _p(perm), code, N, E, top, W, ff,
                            _stream()), "moe_down")
    return SplitSum(parts)


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(h, delta)
    _need(h.dtype == torch.float32 and h.dim() == 2 and tuple(delta.shape) == tuple(h.shape)
          and delta.dtype in DTYPE_CODE, "residual_add: h fp32 [N, H], delta of the same shape")
    _ok(_core().ia_residual_add(_p(h), _p(delta), DTYPE_CODE[delta.dtype], h.shape[0], h.shape[1], _stream()),
        "residual_add")
    return h


def rope_kv_append(qkv, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], nh: int, nkv: int,
                   d: int, rot: int, slots: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
                   v_pages: Optional[torch.Tensor] = None, q_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate q and k, and write k and v to their page slots.  Returns the rotated q, [N, >= nh d].

    qkv is [N, (nh + 2 nkv) d] (or [N, nh d] when no pages are given), a tensor or a :class:`SplitSum`.
    A tensor is rotated in place unless ``q_out`` is given; a SplitSum needs ``q_out`` [N, nh d] (made here
    when absent).  Key pages are [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size].
    """
    split = isinstance(qkv, SplitSum)
    src = qkv.parts if split else qkv
    write = k_pages is not None
    N, row = (src.shape[1], src.shape[2]) if split else tuple(src.shape)
    act = (k_pages.dtype if write else (q_out.dtype if q_out is not None else None)) if split else src.dtype
    _need(act is not None, "rope: partial sums need pages or q_out to tell the activations' dtype")
    if q_out is None:
        q_out = torch.empty((N, nh * d), dtype=act, device=src.device) if split else src
    _dev(src, positions, inv_freq, slots, k_pages, v_pages)
    _need(q_out.is_cuda and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == N
          and q_out.shape[1] >= nh * d and q_out.dtype == act, "rope: q_out must be [N, >= nh*d] in the activations' dtype")
    _need(act in DTYPE_CODE and src.dtype in DTYPE_CODE, "rope: dtype")
    _need(row >= (nh + (2 * nkv if write else 0)) * d, "rope: row of qkv is too short for its heads")
    _i32(positions, N, "rope positions")
    if inv_freq is not None:
        _need(inv_freq.dtype in (torch.float32, torch.float64) and inv_freq.numel() == rot // 2 and rot % 2 == 0
              and 0 < rot <= d, "rope: inv_freq must hold rot/2 fp32 or float64 values, rot even and at most the head size")
    page_size = num_pages = 0
    if write:
        _need(v_pages is not None and slots is not None, "rope: k_pages, v_pages and slots go together")
        _need(k_pages.dtype == act and v_pages.dtype == act, "rope: pages must have the activations' dtype")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
        _need(k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d
              and tuple(v_pages.shape) == (num_pages, nkv, d, page_size),
              "rope: key pages must be [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size]")
        _i32(slots, N, "rope slots")
    _ok(_core().ia_rope_kv_append(_p(src), DTYPE_CODE[src.dtype], src.shape[0] if split else 1, N, _p(q_out),
                                  q_out.stride(0), DTYPE_CODE[act], _p(positions), _p(slots), _p(inv_freq),
                                  1 if (inv_freq is not None and inv_freq.dtype == torch.float64) else 0,
                                  _p(k_pages), _p(v_pages), N, row, nh, nkv, d, rot if inv_freq is not None else 0,
                                  page_size, num_pages, 1 if write else 0, _stream()), "rope_kv_append")
    return q_out


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i]."""
    _dev(gate_up, out)
    N, two_i = gate_up.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (N, two_i // 2) and out.dtype == gate_up.dtype
          and out.dtype in DTYPE_CODE, "swiglu: gate_up [N, 2I] and out [N, I] of one dtype")
    _ok(_core().ia_swiglu(_p(gate_up), _p(out), DTYPE_CODE[out.dtype], N, two_i // 2, _stream()), "swiglu")
    return out


def cast(src: torch.Tensor, dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``src`` in another of the two types (fp32 to bf16 rounds to nearest even; bf16 to fp32 is exact)."""
    _dev(src, out)
    _need(src.dtype in DTYPE_CODE and dtype in DTYPE_CODE, "cast: fp32 and bf16 only")
    if out is None:
        out = torch.empty(src.shape, dtype=dtype, device=src.device)
    _need(out.dtype == dtype and out.numel() == src.numel(), "cast: out must have src's size and the asked type")
    _ok(_core().ia_cast(_p(src), DTYPE_CODE[src.dtype], _p(out), DTYPE_CODE[dtype], ctypes.c_size_t(src.numel()),
                        _stream()), "cast")
    return out


def gather_tokens(token_ids: torch.Tensor, source: torch.Tensor, index: torch.Tensor) -> None:
    """token_ids[i] = source[index[i]] where index[i] >= 0; other places stay.  All int32 on the device."""
    _dev(token_ids, source, index)
    n = token_ids.numel()
    _i32(token_ids, n, "gather_tokens token_ids")
    _i32(index, n, "gather_tokens index")
    _i32(source, 0, "gather_tokens source")
    _ok(_core().ia_gather_tokens(_p(token_ids), _p(source), _p(index), n, source.numel(), _stream()), "gather_tokens")


def words_from_host(dst: torch.Tensor, pinned: torch.Tensor, n: int, token_off: int = 0, nd: int = 0,
                    source: Optional[torch.Tensor] = None, index_off: int = 0) -> None:
    """dst[:n] = pinned[:n] (4-byte words; ``pinned`` in pinned host memory) by a kernel of the current stream;
    with ``nd`` > 0 the words dst[token_off + r], r < nd, whose index pinned[index_off + r] is j >= 0 become
    source[j] (int32 on the device)."""
    _need(dst.is_cuda and dst.is_contiguous() and dst.element_size() == 4 and dst.numel() >= n,
          "words_from_host: a contiguous device tensor of 4-byte elements, at least n long")
    _need(pinned.is_pinned() and pinned.element_size() == 4 and pinned.numel() >= max(n, index_off + nd),
          "words_from_host: the source must be pinned host memory of 4-byte elements, long enough")
    if nd:
        _i32(source, 0, "words_from_host tokens")
    _ok(_core().ia_words_from_host(_p(dst), ctypes.c_void_p(pinned.data_ptr()), int(n), int(token_off), int(nd),
                                   _p(source), source.numel() if source is not None else 0, int(index_off), _stream()),
        "words_from_host")


def words_to_host(pinned: torch.Tensor, src: torch.Tensor) -> None:
    """pinned[:n] = src (4-byte words) by a kernel of the current stream; an event recorded after it tells the
    host when the words are there."""
    n = src.numel()
    _need(src.is_cuda and src.is_contiguous() and src.element_size() == 4, "words_to_host: a device tensor of 4-byte elements")
    _need(pinned.is_pinned() and pinned.element_size() == 4 and pinned.numel() >= n,
          "words_to_host: the target must be pinned host memory of 4-byte elements, long enough")
    _ok(_core().ia_words_to_host(ctypes.c_void_p(pinned.data_ptr()), _p(src), n, _stream()), "words_to_host")


def copy_pages(pool: torch.Tensor, src_pages: torch.Tensor, dst_pages: torch.Tensor) -> None:
    """pool[dst_pages[i]] = pool[src_pages[i]] for a pool [num_pages, ...]; pairs with a page outside the pool
    are left out.  The targets must differ from each other and from every source."""
    _dev(pool, src_pages, dst_pages)
    n = src_pages.numel()
    _need(pool.dim() >= 2 and pool.shape[0] > 0, "copy_pages: a pool [num_pages, ...]")
    _i32(src_pages, n, "copy_pages sources")
    _i32(dst_pages, n, "copy_pages targets")
    page_bytes = pool[0].numel() * pool.element_size()
    _need(page_bytes % 4 == 0 and n <= 65535, "copy_pages: pages of a multiple of 4 bytes, at most 65,535 pairs")
    _ok(_core().ia_copy_pages(_p(pool), ctypes.c_size_t(page_bytes), pool.shape[0], _p(src_pages), _p(dst_pages), n,
                              _stream()), "copy_pages")


# ------------------------------------------------------------------ matrix products
def gemm_generic(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with fp32 multiply-adds in the order of k."""
    _dev(w, out)
    _need(a.is_cuda and a.dim() == 2 and a.stride(1) == 1, "gemm: a must be a GPU matrix with unit inner stride")
    M, K = a.shape
    N = w.shape[0]
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: weight must be [N, {K}], got {tuple(w.shape)}")
    _need(a.dtype == w.dtype and a.dtype in DTYPE_CODE and out.dtype in DTYPE_CODE, "gemm: dtypes")
    _need(tuple(out.shape) == (M, N), f"gemm: out must be [{M}, {N}]")
    lda = a.stride(0) if M > 1 else K
    _need(lda >= K, "gemm: a's rows overlap")
    _ok(_core().ia_gemm_generic(_p(a), _p(w), _p(out), DTYPE_CODE[a.dtype], DTYPE_CODE[out.dtype], M, N, K, lda, K, N,
                                _stream()), "gemm_generic")
    return out


MFMA_GEMM_TILES = {"auto": 0, "256x256": 1, "128x256": 2, "128x128": 3}


def gemm_mfma_supported(M: int, N: int, K: int) -> bool:
    """Sizes the LDS-tiled MFMA product takes: K in steps of 64, rows addressed with 32-bit byte offsets."""
    return M >= 1 and N >= 1 and K >= 64 and K % 64 == 0 and M * K * 2 < 2 ** 32 and N * K * 2 < 2 ** 32


def gemm_mfma(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None, tile: str = "auto") -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T, bf16 with fp32 accumulation, for many rows (prefill): both operands
    tiled through LDS, ``v_mfma_f32_32x32x16_bf16``.  A row of the result depends on its own row of ``a`` only."""
    _dev(a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma: contiguous operands")
    _need(gemm_mfma_supported(M, N, K), f"gemm_mfma: M={M} N={N} K={K} not supported (K % 64 == 0, below 4 GiB)")
    _need(tile in MFMA_GEMM_TILES, f"gemm_mfma: unknown tile {tile!r}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N),
          f"gemm_mfma: out must be contiguous bf16 [{M}, {N}]")
    _ok(_core().ia_gemm_mfma(_p(a), _p(w), _p(out), M, N, K, MFMA_GEMM_TILES[tile], _stream()), "gemm_mfma")
    return out


def gemm_mfma_swiglu(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                     tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(a @ w[:N/2]^T) * (a @ w[N/2:]^T) as bf16 [M, N/2]: the LDS-tiled MFMA product (tiles of 128 x 128) with
    the activation on its fp32 sums in the epilogue, for up to some hundred rows.  ``tiled``: the copy of ``w`` that
    :func:`tile_weight` made with the "swiglu" epilogue, read instead of ``w`` (the same bits)."""
    _dev(a, w, out, tiled)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma_swiglu: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma_swiglu: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma_swiglu: contiguous operands")
    _need(N % 2 == 0 and gemm_mfma_supported(M, N, K),
          f"gemm_mfma_swiglu: M={M} N={N} K={K} not supported (N even, K % 64 == 0, below 4 GiB)")
    if out is None:
        out = torch.empty((M, N // 2), dtype=torch.bfloat16, device=a.device)
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, N // 2),
          f"gemm_mfma_swiglu: out must be contiguous bf16 [{M}, {N // 2}]")
    if tiled is not None:
        _core().ia_gemm_skinny_tiled_elements.restype = ctypes.c_size_t
        _need(tiled.dtype == torch.bfloat16 and tiled.is_contiguous() and gemm_skinny_splits(N, K) == 1 and
              tiled.numel() == int(_core().ia_gemm_skinny_tiled_elements(N, K, EPILOGUE["swiglu"])),
              "gemm_mfma_swiglu: tiled is not the copy, made for the swiglu epilogue, of a weight that is not split over K")
    _ok(_core().ia_gemm_mfma_swiglu(_p(a), _p(tiled if tiled is not None else w), int(tiled is not None), _p(out),
                                    M, N, K, _stream()), "gemm_mfma_swiglu")
    return out


def gemm_mfma_split(a: torch.Tensor, w: torch.Tensor, splits: int, parts: Optional[torch.Tensor] = None) -> SplitSum:
    """a[M, K] @ w[N, K]^T for a few hundred rows as fp32 partial sums [splits, M, N]: the LDS-tiled MFMA product
    with tiles of 128 x 128 and K split over ``splits`` workgroups a tile, so that the launch fills the GPU where the
    tiles alone would not and the weight comes at the memory's rate; the next kernel adds the parts."""
    _dev(a, w, parts)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_mfma_split: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_mfma_split: bf16 operands")
    _need(a.is_contiguous() and w.is_contiguous(), "gemm_mfma_split: contiguous operands")
    _need(gemm_mfma_supported(M, N, K), f"gemm_mfma_split: M={M} N={N} K={K} not supported (K % 64 == 0, below 4 GiB)")
    _need(1 <= splits <= K // 64, f"gemm_mfma_split: {splits} parts of K={K} (1 to K / 64)")
    if parts is None:
        parts = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and tuple(parts.shape) == (splits, M, N),
          f"gemm_mfma_split: parts must be contiguous fp32 [{splits}, {M}, {N}]")
    _ok(_core().ia_gemm_mfma_split(_p(a), _p(w), _p(parts), M, N, K, splits, _stream()), "gemm_mfma_split")
    return SplitSum(parts)


LIBRARY_WORKSPACE_BYTES = 128 << 20
_library_workspace: Dict[torch.device, torch.Tensor] = {}


def library_workspace(device: torch.device) -> torch.Tensor:
    """The one workspace of the library's products on a device."""
    ws = _library_workspace.get(device)
    if ws is None:
        ws = _library_workspace[device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def gemm_library(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T by the vendor's library (hipBLASLt), called directly: bf16 with fp32
    accumulation, or fp32 throughout.  The library's choice of an algorithm is asked once per shape and kept,
    so a later product of the same shape costs one call on the host.  All products share one workspace per
    device: they must be on one stream, or ordered otherwise."""
    _dev(a, w, out)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], "gemm_library: shapes")
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == w.dtype and a.dtype in DTYPE_CODE, "gemm_library: bf16 or fp32 operands of one dtype")
    _need(M >= 1 and N >= 1 and K >= 1, "gemm_library: empty operand")
    if out is None:
        out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    _need(out.dtype == a.dtype and tuple(out.shape) == (M, N), f"gemm_library: out must be {a.dtype} [{M}, {N}]")
    ws = library_workspace(a.device)
    lib = load_library("blaslt")
    code = lib.ia_gemm_lt(_p(a), _p(w), _p(out), M, N, K, DTYPE_CODE[a.dtype], _p(ws), ctypes.c_size_t(ws.numel()),
                          _stream())
    if code == 10003:
        raise KernelError(f"gemm_library: hipBLASLt failed with status {lib.ia_gemm_lt_last_status()} "
                          f"(M={M} N={N} K={K} {a.dtype})")
    _ok(code, f"gemm_library (M={M} N={N} K={K})")
    return out


SKINNY_MAX_M = 128
EPILOGUE = {None: 0, "swiglu": 1}


def gemm_skinny_supported(M: int, N: int, K: int) -> bool:
    return 0 < M <= SKINNY_MAX_M and K % 8 == 0 and K >= 8 and N >= 1


def gemm_skinny_splits(N: int, K: int) -> int:
    """Parts the inner dimension is split into for a weight [N, K] (depends on N and K only)."""
    return int(_core().ia_gemm_skinny_splits(N, K))


def tile_weight(w: torch.Tensor, epilogue: Optional[str] = None) -> torch.Tensor:
    """A copy of the weight [N, K] (bf16) laid out for :func:`gemm_skinny` with this epilogue: the 64 rows x 256
    values that a workgroup multiplies with in one chunk are 32 KB of consecutive memory, chunk after chunk, so
    every workgroup reads one stretch of memory front to back (rows padded to whole workgroups, K to whole chunks,
    with zeros).  Pass it as ``tiled``; the result has the same bits."""
    _dev(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and epilogue in EPILOGUE, "tile_weight: a bf16 matrix [N, K]")
    N, K = w.shape
    lib = _core()
    lib.ia_gemm_skinny_tiled_elements.restype = ctypes.c_size_t
    n = int(lib.ia_gemm_skinny_tiled_elements(N, K, EPILOGUE[epilogue]))
    out = torch.empty(n, dtype=torch.bfloat16, device=w.device)
    _ok(lib.ia_gemm_skinny_tile(_p(w), _p(out), N, K, EPILOGUE[epilogue], _stream()), "tile_weight")
    return out


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
                epilogue: Optional[str] = None, keep_split: bool = False,
                out_dtype: torch.dtype = torch.bfloat16, tiled: Optional[torch.Tensor] = None):
    """a[M, K] @ w[N, K]^T for M <= 64 on MFMA, weights streamed once; bf16 operands, fp32 sums.

    Returns ``out`` ([M, N] bf16 or fp32; [M, N/2] with the "swiglu" epilogue, silu(left half) * right half),
    or, with ``keep_split`` and a product that is split, a :class:`SplitSum` for the next kernel to join.
    """
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bf16 operands")
    _need(w.dim() == 2 and w.shape[1] == K, "gemm_skinny: shapes")
    _need(gemm_skinny_supported(M, N, K), f"gemm_skinny: M={M} N={N} K={K} not supported (M <= 128, K % 8 == 0)")
    _need(epilogue in EPILOGUE, f"gemm_skinny: unknown epilogue {epilogue!r}")
    _need(epilogue is None or N % 2 == 0, "gemm_skinny: the swiglu epilogue needs an even N")
    splits = gemm_skinny_splits(N, K)
    ws = None
    if splits > 1:
        ws = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
    launch, wp = _core().ia_gemm_skinny, _p(w)
    if tiled is not None:
        _need(tiled.is_cuda and tiled.dtype == torch.bfloat16 and tiled.is_contiguous(), "gemm_skinny: the tiled copy")
        launch, wp = _core().ia_gemm_skinny_tiled, _p(tiled)
    if keep_split and epilogue is None and splits > 1:
        _ok(launch(_p(a), wp, None, 0, M, N, K, 0, _p(ws), ctypes.c_size_t(ws.numel()), _stream()), "gemm_skinny")
        return SplitSum(ws)
    n_out = N // 2 if epilogue == "swiglu" else N
    if out is None:
        out = torch.empty((M, n_out), dtype=out_dtype, device=a.device)
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (M, n_out) and out.is_contiguous(),
          f"gemm_skinny: out must be contiguous [{M}, {n_out}]")
    _ok(launch(_p(a), wp, _p(out), DTYPE_CODE[out.dtype], M, N, K, EPILOGUE[epilogue], _p(ws),
               ctypes.c_size_t(ws.numel() if ws is not None else 0), _stream()), "gemm_skinny")
    return out


def gemm_skinny_rows(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T for any M through :func:`gemm_skinny`'s kernel, 128 rows at a time (an fp32
    result from bf16 operands has no other kernel: the head of a step that wants the logits of many places)."""
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == K,
          "gemm_skinny_rows: bf16 operands [M, K] and [N, K]")
    _need(M >= 1 and gemm_skinny_supported(1, N, K), f"gemm_skinny_rows: M={M} N={N} K={K} not supported (K % 8 == 0)")
    _need(out.dtype in DTYPE_CODE and tuple(out.shape) == (M, N), f"gemm_skinny_rows: out must be contiguous [{M}, {N}]")
    splits = gemm_skinny_splits(N, K)
    ws = torch.empty((splits, min(M, SKINNY_MAX_M), N), dtype=torch.float32, device=a.device) if splits > 1 else None
    _ok(_core().ia_gemm_skinny_rows(_p(a), _p(tiled if tiled is not None else w), int(tiled is not None), _p(out),
                                    DTYPE_CODE[out.dtype], M, N, K, _p(ws),
                                    ctypes.c_size_t(ws.numel() if ws is not None else 0), _stream()), "gemm_skinny_rows")
    return out


# ------------------------------------------------------------------------ attention
def _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, what):
    _dev(qkv, k_pages, v_pages, out, block_tables)
    _need(qkv.dtype == out.dtype == k_pages.dtype == v_pages.dtype and qkv.dtype in DTYPE_CODE,
          f"{what}: q, pages and out must share one dtype")
    _need(qkv.dim() == 2 and qkv.shape[1] >= nh * d, f"{what}: q rows must hold nh*d values")
    _need(out.dim() == 2 and out.shape[1] == nh * d and out.shape[0] == qkv.shape[0],
          f"{what}: out must be [N, nh*d]")
    _need(k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d
          and tuple(v_pages.shape) == (k_pages.shape[0], nkv, d, k_pages.shape[2]),
          f"{what}: key pages must be [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2, f"{what}: block_tables int32 [B, MB]")
    _need(nh % nkv == 0, f"{what}: nh must be a multiple of nkv")


def attention_generic(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      token_seq: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor, nh: int,
                      nkv: int, d: int, scale: float, window: int = 0, sinks: Optional[torch.Tensor] = None) -> None:
    """Causal paged attention, one wave per (token, head), fp32 arithmetic.  ``sinks`` fp32 [nh]: exp(sinks[h]) is
    added to the softmax's denominator of head h.

    qkv [N, >= nh*d]: the q heads of token n are the first nh*d values of row n.
    token_seq[n] is the row of block_tables of token n; positions[n] its position.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention")
    N = out.shape[0]
    _i32(token_seq, N, "attention token_seq")
    _i32(positions, N, "attention positions")
    _need(0 < d <= GENERIC_MAX_HEAD_DIM, f"attention: head size must be at most {GENERIC_MAX_HEAD_DIM}")
    _f32(sinks, nh, "attention sinks")
    _ok(_core().ia_attention_generic(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d,
                                     DTYPE_CODE[out.dtype], _p(token_seq), _p(positions), _p(block_tables),
                                     block_tables.shape[1], N, nh, nkv, d, k_pages.shape[2], k_pages.shape[0],
                                     ctypes.c_float(scale), int(window), _p(sinks), _stream()), "attention_generic")


def _attn(d: int) -> ctypes.CDLL:
    lib = load_library(f"attn_d{d}")
    return lib


_compute_units: Dict[int, int] = {}


def compute_units(device: Optional[torch.device] = None) -> int:
    """Compute units of the device (asked once): what the launch shapes below are sized against."""
    idx = device.index if (device is not None and device.index is not None) else torch.cuda.current_device()
    cus = _compute_units.get(idx)
    if cus is None:
        cus = _compute_units[idx] = int(torch.cuda.get_device_properties(idx).multi_processor_count)
    return cus


def decode_splits(batch: int, nh: int, nkv: int, max_len: int, device: Optional[torch.device] = None,
                  head_dim: int = 128) -> int:
    """Parts the keys of a request are cut into, so that a small batch still fills the GPU (workgroups of
    four waves, each wave one tile of 16 keys at a time).  Measured on 256 compute units, with the join's launch:

    * head sizes up to 128: about one workgroup a compute unit while the batch alone gives at most a quarter of
      that, about two up to five eighths, and no parts above that (8B shape, 527 keys: 24 requests 13.9 us whole
      against 15.3 in three parts, 32 requests 15.4 against 17.1 in two); at head sizes up to 64 a tile is half the
      bytes and twice as many workgroups are wanted (8 requests with 32,768 keys each: 97 us in eight parts, 138
      in four; 32 requests: 364 in two, 520 whole);
    * above 128 a compute unit holds one workgroup, and more parts than compute units only cost (head size 256, 32
      requests on 4 key/value heads: 19 us in two parts, 23 in four);
    * the join grows with the parts as the work of a part shrinks with them: the best number of parts for one
      request went with the square root of its tiles (4 parts at 512 keys, 8 at 2,048, 16 at 8,192, 32 at 32,768, for
      head sizes 64, 128 and 256 alike), so that bounds the parts; never more than 64."""
    cus = compute_units(device)
    fill = cus * (2 if head_dim <= 64 else 1)
    groups = batch * nkv * ((nh // nkv + 15) // 16)
    tiles = max(1, (max_len + 15) // 16)
    if 8 * groups >= 5 * fill:
        return 1
    if head_dim > 128:
        wanted = fill // groups
    else:
        wanted = fill // groups if 4 * groups <= fill else 2 * fill // groups
    return max(1, min(wanted, math.isqrt(tiles // 2), 64))


def attention_decode(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                     positions: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                     window: int, max_len: int, num_splits: Optional[int] = None,
                     sinks: Optional[torch.Tensor] = None) -> None:
    """bf16 attention of B single tokens (row b of qkv: token b at positions[b]) over their pages, on MFMA.

    ``max_len`` bounds the positions (host side), and sets how many parts the keys are split into.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention_decode")
    B = out.shape[0]
    _need(qkv.dtype == torch.bfloat16, "attention_decode: bf16 only")
    _i32(positions, B, "attention_decode positions")
    _need(block_tables.shape[0] >= B, "attention_decode: one row of block_tables per token")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_decode: page size {ps} is not a multiple of 4")
    _need(block_tables.shape[1] * ps >= max_len, "attention_decode: block_tables are narrower than max_len")
    splits = num_splits or decode_splits(B, nh, nkv, max_len, out.device, d)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(B * nh * splits * d, dtype=torch.float32, device=out.device)
        part_ml = torch.empty(B * nh * splits * 2, dtype=torch.float32, device=out.device)
    _ok(_attn(d).ia_attn_decode(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d, _p(part_o),
                                _p(part_ml), _p(positions), _p(block_tables), block_tables.shape[1], B, nh, nkv, ps,
                                k_pages.shape[0], ctypes.c_float(scale), int(window), splits, _p(sinks), _stream()),
        "attention_decode")


def attention_decode_rotating(qkv, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot: int,
                              slots: Optional[torch.Tensor], k_pages: torch.Tensor, v_pages: torch.Tensor,
                              out: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, d: int, scale: float,
                              window: int, max_len: int, num_splits: Optional[int] = None,
                              sinks: Optional[torch.Tensor] = None) -> None:
    """:func:`rope_kv_append` and :func:`attention_decode` of B single tokens in one launch (the same bits).

    ``qkv`` is the QKV product of the tokens, [B, (nh + 2 nkv) d] in bf16 or a :class:`SplitSum` of it (with
    ``slots`` None only the nh query heads are read and no key or value is made: the pages belong to another
    run of a layer).  Rotated queries stay inside the kernel; the token's key and value go to their slot of the
    pages and take part in the attention.
    """
    split = isinstance(qkv, SplitSum)
    src = qkv.parts if split else qkv
    B = out.shape[0]
    rows, row = (src.shape[1], src.shape[2]) if split else tuple(src.shape)
    _need(src.is_cuda and src.is_contiguous(), "attention_decode_rotating: qkv must be contiguous on the GPU")
    _need(src.dtype == (torch.float32 if split else torch.bfloat16),
          "attention_decode_rotating: bf16 rows or fp32 partial sums")
    _need(rows >= B and row >= (nh + (2 * nkv if slots is not None else 0)) * d,
          "attention_decode_rotating: rows of qkv are too few or too short for their heads")
    _need(k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
          and k_pages.dim() == 4 and k_pages.shape[1] == nkv and k_pages.shape[3] == d and out.is_cuda
          and tuple(v_pages.shape) == (k_pages.shape[0], nkv, d, k_pages.shape[2]) and tuple(out.shape) == (B, nh * d)
          and out.is_contiguous() and k_pages.is_contiguous() and v_pages.is_contiguous(),
          "attention_decode_rotating: bf16 key pages [num_pages, nkv, page_size, d], value pages "
          "[num_pages, nkv, d, page_size], out [B, nh d]")
    _dev(src, positions, inv_freq, slots, k_pages, v_pages, out, block_tables)
    _i32(positions, B, "attention_decode_rotating positions")
    if slots is not None:
        _i32(slots, B, "attention_decode_rotating slots")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
          and block_tables.shape[0] >= B, "attention_decode_rotating: one int32 row of block_tables per token")
    if inv_freq is not None:
        _need(inv_freq.dtype in (torch.float32, torch.float64) and inv_freq.numel() == rot // 2 and rot % 2 == 0
              and 0 < rot <= d and inv_freq.is_contiguous(),
              "attention_decode_rotating: inv_freq must hold rot/2 fp32 or float64 values, rot even and at most d")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_decode_rotating: page size {ps} is not a multiple of 4")
    _need(block_tables.shape[1] * ps >= max_len, "attention_decode_rotating: block_tables are narrower than max_len")
    splits = num_splits or decode_splits(B, nh, nkv, max_len, out.device, d)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(B * nh * splits * d, dtype=torch.float32, device=out.device)
        part_ml = torch.empty(B * nh * splits * 2, dtype=torch.float32, device=out.device)
    _ok(_attn(d).ia_attn_decode_fused(
        _p(src), DTYPE_CODE[src.dtype], src.shape[0] if split else 1, rows, row, _p(slots), _p(inv_freq),
        1 if (inv_freq is not None and inv_freq.dtype == torch.float64) else 0, rot if inv_freq is not None else 0,
        _p(k_pages), _p(v_pages), _p(out), nh * d, _p(part_o), _p(part_ml), _p(positions), _p(block_tables),
        block_tables.shape[1], B, nh, nkv, ps, k_pages.shape[0], ctypes.c_float(scale), int(window), splits, _p(sinks),
        _stream()), "attention_decode_rotating")


PREFILL_TILE_ROWS = 64      # query rows of a workgroup's tile in attention_prefill
PREFILL_PAIRED = 0x100      # in a launch shape: 32 rows from each end of a request in place of 64 consecutive ones


def attention_prefill(qkv: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      seq_starts: torch.Tensor, seq_ctx: torch.Tensor, block_tables: torch.Tensor,
                      tiles: torch.Tensor, num_tiles: int, nh: int, nkv: int, d: int, scale: float,
                      window: int, heads_per_workgroup: int = 0, paired: bool = False,
                      sinks: Optional[torch.Tensor] = None) -> None:
    """bf16 causal attention of portions of prompts over their pages, on MFMA.

    Request s brings rows seq_starts[s] .. seq_starts[s+1]-1 of qkv and had seq_ctx[s] tokens cached
    before; tiles[i] = (s, first row of a block of PREFILL_TILE_ROWS among the request's rows).  ``heads_per_workgroup``:
    0 for the kernel's own choice, or 1, 2, 4; ``paired``: a workgroup takes half a block of rows from each end of
    its request's new tokens, so that all workgroups of a request have the same work under the causal mask (every
    block of every request must be listed then; without effect under a window).  A value of :func:`prefill_launch_shape` may stand in
    ``heads_per_workgroup`` for both.  The result has the same bits whatever the shape.
    """
    _check_paged(qkv, k_pages, v_pages, out, block_tables, nh, nkv, d, "attention_prefill")
    _need(qkv.dtype == torch.bfloat16, "attention_prefill: bf16 only")
    B = block_tables.shape[0]
    _i32(seq_starts, B + 1, "attention_prefill seq_starts")
    _i32(seq_ctx, B, "attention_prefill seq_ctx")
    _need(tiles.dtype == torch.int32 and tiles.is_cuda and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles,
          "attention_prefill: tiles int32 [num_tiles, 2]")
    ps = k_pages.shape[2]
    _need(ps % 4 == 0, f"attention_prefill: page size {ps} is not a multiple of 4")
    _ok(_attn(d).ia_attn_prefill(_p(qkv), qkv.shape[1], _p(k_pages), _p(v_pages), _p(out), nh * d, _p(seq_starts),
                                 _p(seq_ctx), _p(block_tables), block_tables.shape[1], _p(tiles), num_tiles, nh, nkv,
                                 ps, k_pages.shape[0], ctypes.c_float(scale), int(window),
                                 int(heads_per_workgroup) | (PREFILL_PAIRED if paired else 0), _p(sinks), _stream()),
        "attention_prefill")


def prefill_launch_shape(nh: int, nkv: int, d: int, q_lens: Sequence[int], ctx_lens: Sequence[int],
                         window: int, device: torch.device) -> int:
    """The shape of the :func:`attention_prefill` launch for these portions of prompts (``q_lens`` new tokens
    after ``ctx_lens`` cached ones each): how many query heads share a workgroup's tiles of keys (0: the kernel's
    default), with :data:`PREFILL_PAIRED` added when a workgroup should take half its rows from each end of its
    request.  The bits of the result do not depend on it; all figures are of the 8B shape (32 heads over 8, 128).

    Four heads a workgroup (the default at head sizes 80 to 160 with three or more query heads to a key/value
    head) read the keys least often but make few workgroups: when they would fill fewer than three quarters of
    the compute units, two heads are taken (1,024 tokens: 34 against 49 us).  When the launch has no more
    workgroups than compute units, every workgroup runs from start to end and the longest sets the time: under
    the causal mask that is the last block of a prompt, with twice the rounds of the average one.  Paired rows
    give all workgroups of a request the same work then (2,048 tokens: 66 against 89 us with four heads, 71 with
    two unpaired; 2,048 after 2,048: 147 against 171).  With more workgroups than compute units the rounds of a
    paired workgroup in which half its waves have run out of keys cost more than the balance gains (4,096
    tokens: 220 against 192 us), and under a window the rows of the two ends share no keys: not paired then.
    """
    G = nh // nkv
    widest = 4 if 80 <= d <= 160 else 2
    hpw = widest if G >= 3 else (2 if G == 2 else 1)
    tiles = total = longest = 0
    for q, c in zip(q_lens, ctx_lens):
        for first in range(0, q, 64):           # a block of 64 rows sees the keys up to its last row, or a window's worth
            keys = c + min(q, first + 64)
            if window:                          # a sliding window, or (negative) chunks of that many positions
                keys = min(keys, abs(window) + 64)
            tiles += 1
            total += keys
            longest = max(longest, keys)
    if tiles == 0:
        return 0
    cus = compute_units(device)
    workgroups = tiles * nkv * ((G + hpw - 1) // hpw)
    if hpw == 4 and 4 * workgroups < 3 * cus:
        hpw, workgroups = 2, tiles * nkv * ((G + 1) // 2)
    if window == 0:
        return hpw | (PREFILL_PAIRED if workgroups <= cus else 0)
    # under a window: two heads where four would give at most one workgroup a compute unit with the longest
    # block at 1.5 times the average (more, smaller workgroups fill what the long ones leave idle)
    if hpw == 4 and workgroups <= cus and longest * tiles >= 1.5 * total:
        hpw = 2
    return hpw


# ------------------------------------------------------------- mixers with a little state from token to token
CONV_ACTIVATIONS = {None: 0, "silu": 1}
PAIRINGS = {"half": 0, "neighbours": 1}


def _f32(t: Optional[torch.Tensor], n: int, what: str) -> None:
    if t is not None:
        _need(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n, f"{what}: {n} fp32 values")


def _rows(t: torch.Tensor, cols: int, what: str) -> None:
    _need(t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.shape[1] >= cols and t.dtype in DTYPE_CODE,
          f"{what}: rows of at least {cols} values, fp32 or bf16")


def _state_rows(state: torch.Tensor, need: int, what: str) -> int:
    """``state`` [slots, per slot] fp32, a slot's values consecutive: the slot's stride in floats."""
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= need, f"{what}: state [slots, >= {need}] fp32")
    return int(state.stride(0))


def causal_conv(u: torch.Tensor, w: torch.Tensor, state: torch.Tensor, ctx_token_seq: torch.Tensor,
                seq_starts: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                bias_in: Optional[torch.Tensor] = None, bias_out: Optional[torch.Tensor] = None,
                activation: Optional[str] = None, tap_major: bool = False) -> torch.Tensor:
    """out[t, c] = act(bias_out[c] + sum_j w[c, j] (u[t - (taps-1) + j, c] + bias_in[c])) over each request's own
    tokens; the inputs before this step's rows come from ``state`` [slots, >= (taps-1) C] fp32 (the request's last
    taps-1 inputs, zero before its start).  ``u`` and ``out`` may be column ranges of wider rows.  The state is
    left as it was: :func:`conv_state_update` moves it on.  ``tap_major``: ``w`` is stored [taps, C], which lets
    bf16 rows of whole 16-byte pieces run eight channels a thread."""
    N, (C, taps) = u.shape[0], (w.shape[::-1] if tap_major else w.shape)
    _rows(u, C, "causal_conv input")
    _rows(out, C, "causal_conv output")
    _need(out.shape[0] == N and u.shape[1] == C and out.shape[1] == C, "causal_conv: u and out are [N, C]")
    _f32(w, C * taps, "causal_conv weight")
    _f32(bias_in, C, "causal_conv input bias")
    _f32(bias_out, C, "causal_conv output bias")
    stride = _state_rows(state, (taps - 1) * C, "causal_conv")
    _i32(ctx_token_seq, N, "causal_conv token_seq")
    _ok(_core().ia_causal_conv(_p(u), DTYPE_CODE[u.dtype], u.stride(0), _p(bias_in), _p(w), _p(bias_out),
                               CONV_ACTIVATIONS[activation], _p(out), DTYPE_CODE[out.dtype], out.stride(0), _p(state),
                               ctypes.c_long(stride), _p(ctx_token_seq), _p(seq_starts), _p(state_slots), N, C, taps,
                               int(bool(tap_major)), _stream()), "causal_conv")
    return out


def causal_conv_single(u: torch.Tensor, w: torch.Tensor, state: torch.Tensor, ctx_token_seq: torch.Tensor,
                       state_slots: torch.Tensor, out: torch.Tensor, bias_in: Optional[torch.Tensor] = None,
                       bias_out: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                       tap_major: bool = False) -> torch.Tensor:
    """:func:`causal_conv` and :func:`conv_state_update` in one pass for a step in which every request brings exactly
    one token (row r belongs to request ``ctx_token_seq[r]``): the same bits, and the state is left moved on."""
    N, (C, taps) = u.shape[0], (w.shape[::-1] if tap_major else w.shape)
    _rows(u, C, "causal_conv_single input")
    _rows(out, C, "causal_conv_single output")
    _need(out.shape[0] == N and u.shape[1] == C and out.shape[1] == C, "causal_conv_single: u and out are [N, C]")
    _f32(w, C * taps, "causal_conv_single weight")
    _f32(bias_in, C, "causal_conv_single input bias")
    _f32(bias_out, C, "causal_conv_single output bias")
    stride = _state_rows(state, (taps - 1) * C, "causal_conv_single")
    _i32(ctx_token_seq, N, "causal_conv_single token_seq")
    _need(state_slots.numel() >= N, "causal_conv_single: a slot for every row's request")
    _ok(_core().ia_causal_conv_single(_p(u), DTYPE_CODE[u.dtype], u.stride(0), _p(bias_in), _p(w), _p(bias_out),
                                      CONV_ACTIVATIONS[activation], _p(out), DTYPE_CODE[out.dtype], out.stride(0),
                                      _p(state), ctypes.c_long(stride), _p(ctx_token_seq), _p(state_slots), N, C, taps,
                                      int(bool(tap_major)), _stream()), "causal_conv_single")
    return out


def conv_state_update(u: torch.Tensor, taps: int, state: torch.Tensor, seq_starts: torch.Tensor,
                      state_slots: torch.Tensor, bias_in: Optional[torch.Tensor] = None) -> None:
    """After :func:`causal_conv`: every request's state becomes its last taps-1 inputs, this step's included."""
    C, B = u.shape[1], state_slots.numel()
    _rows(u, C, "conv_state_update input")
    _f32(bias_in, C, "conv_state_update input bias")
    stride = _state_rows(state, (taps - 1) * C, "conv_state_update")
    _need(seq_starts.numel() >= B + 1, "conv_state_update: seq_starts holds B + 1 rows")
    _ok(_core().ia_conv_state_update(_p(u), DTYPE_CODE[u.dtype], u.stride(0), _p(bias_in), _p(state),
                                     ctypes.c_long(stride), _p(seq_starts), _p(state_slots), B, C, int(taps), _stream()),
        "conv_state_update")


def qk_prepare(x: torch.Tensor, q_out: torch.Tensor, nh: int, nkv: int, d: int, positions: torch.Tensor,
               q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None, eps: float = 0.0,
               freq: Optional[torch.Tensor] = None, rot: int = 0, pairing: str = "half", magnitude: float = 1.0,
               slots: Optional[torch.Tensor] = None, k_pages: Optional[torch.Tensor] = None,
               v_pages: Optional[torch.Tensor] = None, values_are_keys: bool = False) -> torch.Tensor:
    """Query and key heads between projection and attention.  ``x`` [N, (nh + nkv (+ nkv)) d]: nh query heads,
    nkv key heads, and nkv value heads unless ``values_are_keys`` (then a key head as it comes in is its value).
    Per head: RMS norm over d with one weight for all heads (when given), rotation of the first ``rot`` values
    (``pairing`` "half": value i with i + rot/2; "neighbours": 2i with 2i+1) with sine and cosine times
    ``magnitude``.  Queries go to ``q_out`` [N, nh d], keys and values to their pages at ``slots``."""
    N = x.shape[0]
    write = k_pages is not None
    _rows(x, (nh + (nkv if values_are_keys else 2 * nkv) * int(write)) * d, "qk_prepare input")
    _rows(q_out, nh * d, "qk_prepare q_out")
    _need(q_out.dtype == x.dtype and q_out.shape[0] == N, "qk_prepare: q_out [N, nh d] of the input's dtype")
    _f32(q_norm, d, "qk_prepare q_norm")
    _f32(k_norm, d, "qk_prepare k_norm")
    _i32(positions, N, "qk_prepare positions")
    if rot:
        _need(freq is not None and freq.is_cuda and freq.dtype in (torch.float32, torch.float64)
              and freq.numel() == rot // 2 and rot % 2 == 0 and rot <= d, "qk_prepare: rot/2 frequencies, rot even, <= d")
    ps = num_pages = 0
    if write:
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        _need(slots is not None and v_pages is not None and k_pages.dtype == x.dtype and v_pages.dtype == x.dtype
              and tuple(k_pages.shape) == (num_pages, nkv, ps, d) and tuple(v_pages.shape) == (num_pages, nkv, d, ps)
              and k_pages.is_contiguous() and v_pages.is_contiguous(),
              "qk_prepare: key pages [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d, page_size]")
        _i32(slots, N, "qk_prepare slots")
    _ok(_core().ia_qk_prepare(_p(x), DTYPE_CODE[x.dtype], x.stride(0), _p(q_out), q_out.stride(0), _p(q_norm), _p(k_norm),
                              ctypes.c_float(eps), _p(positions), _p(slots), _p(freq if rot else None),
                              1 if (rot and freq.dtype == torch.float64) else 0, int(rot), PAIRINGS[pairing],
                              ctypes.c_float(magnitude), _p(k_pages), _p(v_pages), N, nh, nkv if write else 0, d, ps,
                              num_pages, int(bool(values_are_keys)), _stream()), "qk_prepare")
    return q_out


def ssd_scan(xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, skip: torch.Tensor,
             state: torch.Tensor, y: torch.Tensor, seq_starts: torch.Tensor, state_slots: torch.Tensor, nh: int, P: int,
             Ns: int, G: int) -> torch.Tensor:
    """Per request and head, over the request's rows in order:  dt = softplus(dt_raw + dt_bias),
    S <- exp(-exp(a_log) dt) S + dt B x^T,  y = S^T C + skip x.  ``xbc`` rows [x: nh P | B: G Ns | C: G Ns];
    ``state`` [slots, >= nh Ns P] fp32 is read and left moved on; ``y`` [N, nh P] fp32."""
    N, B = xbc.shape[0], state_slots.numel()
    _rows(xbc, nh * P + 2 * G * Ns, "ssd_scan xbc")
    _rows(dt_raw, nh, "ssd_scan dt")
    _need(dt_raw.dtype == xbc.dtype and dt_raw.shape[0] == N, "ssd_scan: dt rows of xbc's dtype")
    for t, what in ((dt_bias, "dt_bias"), (a_log, "a_log"), (skip, "skip")):
        _f32(t, nh, "ssd_scan " + what)
    _need(y.is_cuda and y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (N, nh * P),
          "ssd_scan: y [N, nh P] fp32")
    stride = _state_rows(state, nh * Ns * P, "ssd_scan")
    _ok(_core().ia_ssd_scan(_p(xbc), DTYPE_CODE[xbc.dtype], xbc.stride(0), _p(dt_raw), dt_raw.stride(0), _p(dt_bias),
                            _p(a_log), _p(skip), _p(state), ctypes.c_long(stride), _p(y), _p(seq_starts), _p(state_slots),
                            B, nh, P, Ns, G, _stream()), "ssd_scan")
    return y


# tokens of portions in a step from which the recurrence runs as matrix products over chunks
SSD_CHUNKED_FROM = 64


def ssd_chunked_takes(dtype: torch.dtype, nh: int, P: int, Ns: int, G: int, xbc_stride: int) -> bool:
    """Whether :func:`ssd_chunked` has a kernel for these sizes: bf16 rows, P a multiple of 16, a state of a multiple
    of 16 up to 128."""
    return dtype == torch.bfloat16 and bool(_core().ia_ssd_chunked_takes(int(nh), int(P), int(Ns), int(G), int(xbc_stride)))


def ssd_chunked(xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, skip: torch.Tensor,
                state: torch.Tensor, y: torch.Tensor, seq_starts: torch.Tensor, state_slots: torch.Tensor, nh: int, P: int,
                Ns: int, G: int) -> torch.Tensor:
    """What :func:`ssd_scan` computes, as matrix products over chunks of 64 tokens of every request (fp32 but for the
    product of C with B, whose bf16 operands are the stored values): for steps with portions of prompts.  The sums
    are taken in another order than token after token, so results differ from :func:`ssd_scan` by fp32 rounding."""
    N, B = xbc.shape[0], state_slots.numel()
    _rows(xbc, nh * P + 2 * G * Ns, "ssd_chunked xbc")
    _rows(dt_raw, nh, "ssd_chunked dt")
    _need(dt_raw.dtype == xbc.dtype and dt_raw.shape[0] == N, "ssd_chunked: dt rows of xbc's dtype")
    _need(ssd_chunked_takes(xbc.dtype, nh, P, Ns, G, xbc.stride(0)), "ssd_chunked: sizes that it does not take")
    for t, what in ((dt_bias, "dt_bias"), (a_log, "a_log"), (skip, "skip")):
        _f32(t, nh, "ssd_chunked " + what)
    _need(y.is_cuda and y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (N, nh * P),
          "ssd_chunked: y [N, nh P] fp32")
    stride = _state_rows(state, nh * Ns * P, "ssd_chunked")
    _ok(_core().ia_ssd_chunked(_p(xbc), DTYPE_CODE[xbc.dtype], xbc.stride(0), _p(dt_raw), dt_raw.stride(0), _p(dt_bias),
                               _p(a_log), _p(skip), _p(state), ctypes.c_long(stride), _p(y), _p(seq_starts),
                               _p(state_slots), B, nh, P, Ns, G, _stream()), "ssd_chunked")
    return y


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                     out: torch.Tensor) -> torch.Tensor:
    """out = unit_rms(y * silu(z)) * w, the root mean square taken over each of ``groups`` equal parts of a row."""
    N, inner = y.shape
    _need(y.is_cuda and y.dtype == torch.float32 and y.is_contiguous(), "gated_group_norm: y [N, inner] fp32")
    _rows(z, inner, "gated_group_norm gate")
    _f32(w, inner, "gated_group_norm weight")
    _need(out.is_cuda and out.is_contiguous() and tuple(out.shape) == (N, inner) and out.dtype == z.dtype
          and inner % groups == 0, "gated_group_norm: out [N, inner] of the gate's dtype, inner a multiple of groups")
    _ok(_core().ia_gated_group_norm(_p(y), _p(z), DTYPE_CODE[z.dtype], z.stride(0), _p(w), _p(out), N, inner, int(groups),
                                    ctypes.c_float(eps), _stream()), "gated_group_norm")
    return out


def concat_cast(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[N, 2 W] rows [cast(a) | b]: a fp32 [N, W], b [N, W] in the result's dtype."""
    N, W = a.shape
    _need(a.is_cuda and a.dtype == torch.float32 and a.is_contiguous() and b.is_cuda and b.is_contiguous()
          and tuple(b.shape) == (N, W) and b.dtype in DTYPE_CODE, "concat_cast: a fp32 [N, W], b [N, W]")
    if out is None:
        out = torch.empty((N, 2 * W), dtype=b.dtype, device=b.device)
    _need(out.is_contiguous() and tuple(out.shape) == (N, 2 * W) and out.dtype == b.dtype, "concat_cast: out [N, 2 W]")
    _ok(_core().ia_concat_cast(_p(a), _p(b), _p(out), DTYPE_CODE[b.dtype], N, W, _stream()), "concat_cast")
    return out


def stream_add(h: torch.Tensor, delta) -> torch.Tensor:
    """h [N, H] fp32 += delta: a tensor [N, H], or a :class:`SplitSum` whose parts are added in the order of their index."""
    parts = delta.parts if isinstance(delta, SplitSum) else delta
    splits = parts.shape[0] if isinstance(delta, SplitSum) else 1
    _need(h.is_cuda and h.dtype == torch.float32 and h.is_contiguous() and parts.is_cuda and parts.is_contiguous()
          and parts.dtype in DTYPE_CODE and parts.numel() == splits * h.numel(), "stream_add: h fp32 [N, H], delta of its shape")
    _ok(_core().ia_stream_add(_p(h), _p(parts), DTYPE_CODE[parts.dtype], splits, h.shape[0], h.shape[1], _stream()),
        "stream_add")
    return h


def stream_add2(h: torch.Tensor, a, b=None, x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h [N, H] fp32 += a, then += b (each a tensor [N, H] or a :class:`SplitSum`; b may be None), in that order, in one
    pass; ``x`` ([N, H], either type) gets the new h."""
    def parts_of(d):
        return (d.parts, d.parts.shape[0]) if isinstance(d, SplitSum) else (d, 1)
    pa, sa = parts_of(a)
    pb, sb = parts_of(b) if b is not None else (None, 1)
    _need(h.is_cuda and h.dtype == torch.float32 and h.is_contiguous() and pa.is_cuda and pa.is_contiguous()
          and pa.dtype in DTYPE_CODE and pa.numel() == sa * h.numel(), "stream_add2: h fp32 [N, H], a of its shape")
    if pb is not None:
        _need(pb.is_cuda and pb.is_contiguous() and pb.dtype in DTYPE_CODE and pb.numel() == sb * h.numel(),
              "stream_add2: b of h's shape")
    if x is not None:
        _need(x.is_cuda and x.is_contiguous() and x.dtype in DTYPE_CODE and x.shape == h.shape, "stream_add2: x like h")
    _ok(_core().ia_stream_add2(_p(h), _p(pa), DTYPE_CODE[pa.dtype], sa, _p(pb), DTYPE_CODE[pb.dtype] if pb is not None else 0,
                               sb, _p(x), DTYPE_CODE[x.dtype] if x is not None else 0, h.shape[0], h.shape[1], _stream()),
        "stream_add2")
    return h


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y [N, C] += bias [C] (fp32), in place."""
    _need(y.is_cuda and y.is_contiguous() and y.dim() == 2 and y.dtype in DTYPE_CODE, "add_bias: y [N, C]")
    _f32(bias, y.shape[1], "add_bias bias")
    _ok(_core().ia_add_bias(_p(y), DTYPE_CODE[y.dtype], _p(bias), y.shape[0], y.shape[1], _stream()), "add_bias")
    return y


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap tanh(logits / cap), fp32 in place."""
    _need(logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and logits.dim() == 2 and cap > 0,
          "softcap: logits fp32 [R, V], cap positive")
    _ok(_core().ia_softcap(_p(logits), logits.shape[0], logits.shape[1], ctypes.c_float(cap), _stream()), "softcap")
    return logits


def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    """x [R, C] fp32 <- x * s, in place."""
    _need(x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2, "scale_: x fp32 [R, C]")
    _ok(_core().ia_scale(_p(x), x.shape[0], x.shape[1], ctypes.c_float(s), _stream()), "scale_")
    return x


# ------------------------------------------------- gated branches, linear attention, attention with sigmoid weights
def add_rows(h: torch.Tensor, table: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """h [N, H] fp32 += table[index[n]] row by row (a learned vector per position); an index outside the table
    leaves NaN."""
    _dev(h, table, index)
    N, H = h.shape
    _need(h.dtype == torch.float32 and table.dim() == 2 and table.shape[1] == H and table.dtype in DTYPE_CODE,
          "add_rows: h fp32 [N, H], table [rows, H]")
    _i32(index, N, "add_rows index")
    _ok(_core().ia_add_rows(_p(h), _p(table), DTYPE_CODE[table.dtype], _p(index), N, H, table.shape[0], _stream()),
        "add_rows")
    return h


def gated_norm_add(h: torch.Tensor, delta, gate, gate_bias: Optional[torch.Tensor],
                   weight: torch.Tensor, eps: float, next_weight: Optional[torch.Tensor] = None,
                   x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d = delta * sigmoid(gate + gate_bias);  h += d * rsqrt(mean(d^2) + eps) * weight  (fp32, in place).  ``delta``: a
    tensor of h's shape in the activations' dtype or a :class:`SplitSum`; ``gate``: rows of at least H values (fp32 or
    the activations' dtype), a :class:`SplitSum` of the logits, or None for no gate; ``x`` (optional, h's shape in the activations' dtype) receives
    rms_norm(h) * next_weight, or the new h itself without ``next_weight``."""
    split = isinstance(delta, SplitSum)
    d = delta.parts if split else delta
    _dev(h, d, weight, x, gate_bias, next_weight)
    _need(h.dtype == torch.float32 and h.dim() == 2, "gated_norm_add: h must be fp32 [N, H]")
    N, H = h.shape
    splits, d_rows = 1, N
    if split:
        _need(d.shape[1] >= N and d.shape[2] == H, "gated_norm_add: partial sums must be [S, >= N, H]")
        splits, d_rows = d.shape[0], d.shape[1]
    else:
        _need(d is not None and d.dtype in DTYPE_CODE and tuple(d.shape) == (N, H), "gated_norm_add: delta of h's shape")
    g_splits, g_rows = 1, 0
    if isinstance(gate, SplitSum):
        gate = gate.parts
        _need(gate.is_cuda and gate.shape[1] >= N and gate.shape[2] == H, "gated_norm_add: the gate's partial sums must be [S, >= N, H]")
        g_splits, g_rows, g_stride = gate.shape[0], gate.shape[1], H
    elif gate is not None:
        _rows(gate, H, "gated_norm_add gate")
        _need(gate.shape[0] >= N, "gated_norm_add: a gate row per row of h")
        g_rows, g_stride = gate.shape[0], int(gate.stride(0))
    _f32(gate_bias, H, "gated_norm_add gate bias")
    for wt in (weight, next_weight):
        _need(wt is None or (wt.dtype in DTYPE_CODE and wt.numel() == H), f"gated_norm_add: weights of {H} values")
    act = x.dtype if x is not None else (torch.bfloat16 if d.dtype == torch.bfloat16 else torch.float32)
    if x is not None:
        _need(x.dtype in DTYPE_CODE and tuple(x.shape) == (N, H) and (split or x.dtype == d.dtype),
              "gated_norm_add: x of h's shape in the activations' dtype")
    _ok(_core().ia_gated_norm_add(
        _p(h), _p(d), DTYPE_CODE[d.dtype], splits, d_rows, _p(gate), DTYPE_CODE[gate.dtype] if gate is not None else 0,
        g_stride if gate is not None else 0, g_splits, g_rows, _p(gate_bias), _p(weight), DTYPE_CODE[weight.dtype],
        _p(next_weight), DTYPE_CODE[next_weight.dtype] if next_weight is not None else 0, _p(x), DTYPE_CODE[act], N, H,
        ctypes.c_float(eps), _stream()), "gated_norm_add")
    return h


def router_softmax_topk(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int):
    """-> (ids int32 [N, top], weights fp32 [N, top]): s = softmax(logits) over all experts; the ``top`` largest of
    s + correction are chosen (the lowest index among equals); the weights are the chosen s over their sum."""
    _dev(logits, correction)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "router_softmax_topk: fp32 logits [N, E]")
    N, E = logits.shape
    _need(0 < top <= E, f"router_softmax_topk: top must be 1 .. {E}")
    _need(correction is None or (correction.dtype in DTYPE_CODE and correction.numel() == E),
          f"router_softmax_topk: {E} corrections")
    ids = torch.empty((N, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((N, top), dtype=torch.float32, device=logits.device)
    _ok(_core().ia_router_softmax_topk(_p(logits), _p(correction),
                                       DTYPE_CODE[correction.dtype] if correction is not None else 0, _p(ids),
                                       _p(weights), N, E, top, _stream()), "router_softmax_topk")
    return ids, weights


def moe_plain_experts(x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_up: torch.Tensor,
                      w_down: torch.Tensor, act: str, parts: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The chosen experts of every token, each down(act(up x)) without a gate: w_up [E, ff, W], w_down [E, W, ff].
    Fills parts[:top] of fp32 ``parts`` [>= top, N, W], each already times its routing weight, and returns parts."""
    _dev(x, ids, weights, w_up, w_down, parts)
    N, W = x.shape
    E, ff, _ = w_up.shape
    top = ids.shape[1]
    _need(act in ACTIVATIONS, f"moe: unknown activation {act!r}")
    _need(x.dtype in DTYPE_CODE and w_up.dtype == x.dtype and w_down.dtype == x.dtype, "moe: one dtype")
    _need(tuple(w_up.shape) == (E, ff, W) and tuple(w_down.shape) == (E, W, ff), "moe: weights' shapes")
    _need(ids.dtype == torch.int32 and tuple(ids.shape) == (N, top) and weights.dtype == torch.float32
          and tuple(weights.shape) == (N, top), "moe: ids int32 and weights fp32 [N, top]")
    if parts is None:
        parts = torch.empty((top, N, W), dtype=torch.float32, device=x.device)
    _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[0] >= top and tuple(parts.shape[1:]) == (N, W),
          "moe: parts fp32 [>= top, N, W]")
    P = N * top
    offsets = torch.empty(E + 1, dtype=torch.int32, device=x.device)
    perm = torch.empty(max(P, 1), dtype=torch.int32, device=x.device)
    y = torch.empty((max(P, 1), ff), dtype=x.dtype, device=x.device)
    code = DTYPE_CODE[x.dtype]
    _ok(_core().ia_moe_sort(_p(ids), _p(offsets), _p(perm), P, E, _stream()), "moe_sort")
    if moe_grouped_rows(N, E, top, W, ff, x.dtype):
        xs = torch.empty((P, W), dtype=x.dtype, device=x.device)
        _ok(_core().ia_moe_gather(_p(x), _p(perm), _p(xs), P, top, W, _stream()), "moe_gather")
        gemm_mfma_grouped(xs, w_up, offsets, y)
        activation(y, act)
        gemm_mfma_grouped(y, w_down, offsets, xs)
        _ok(_core().ia_moe_scatter(_p(xs), _p(perm), _p(weights), _p(parts), N, top, W, _stream()), "moe_scatter")
        return parts
    _ok(_core().ia_moe_up(_p(x), _p(w_up), _p(y), _p(offsets), _p(perm), code, P, E, top, W, ff, ACTIVATIONS[act],
                          _stream()), "moe_up")
    _ok(_core().ia_moe_down(_p(y), _p(w_down), _p(parts), _p(weights), _p(offsets), _p(perm), code, N, E, top, W, ff,
                            _stream()), "moe_down")
    return parts


def gla_state_floats(nh: int, dim: int, vdim: int) -> int:
    """Floats of a request's state for one run of a gated-linear-attention layer (the heads' S in the kernel's slices)."""
    PW = 16
    return nh * ((vdim + PW - 1) // PW) * dim * PW


def gla_scan(proj: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, z_bias: Optional[torch.Tensor],
             tau: float, q_scale: float, state: torch.Tensor, out: torch.Tensor, seq_starts: torch.Tensor,
             state_slots: torch.Tensor, nh: int, dim: int, vdim: int) -> torch.Tensor:
    """Per request and head over the request's rows in order: alpha = sigmoid(z + z_bias)^(1/tau) per key channel,
    S <- diag(alpha) S + k v^T, out = S^T (q_scale q).  ``proj`` rows hold q and k (nh dim values from q_col, k_col)
    and v (nh vdim from v_col); ``z`` fp32 [N, nh dim]; ``state`` [slots, >= gla_state_floats] fp32 is read and left
    moved on; ``out`` fp32 [N, nh vdim]."""
    N, B = proj.shape[0], state_slots.numel()
    _rows(proj, max(q_col + nh * dim, k_col + nh * dim, v_col + nh * vdim), "gla_scan rows")
    _need(z.is_cuda and z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1 and z.shape[1] >= nh * dim
          and z.shape[0] == N, "gla_scan: z fp32 [N, nh dim]")
    _f32(z_bias, nh * dim, "gla_scan bias")
    _need(out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (N, nh * vdim),
          "gla_scan: out [N, nh vdim] fp32")
    _i32(seq_starts, B + 1, "gla_scan seq_starts")
    _i32(state_slots, B, "gla_scan state_slots")
    stride = _state_rows(state, gla_state_floats(nh, dim, vdim), "gla_scan")
    _ok(_core().ia_gla_scan(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), q_col, k_col, v_col, _p(z),
                            int(z.stride(0)), _p(z_bias), ctypes.c_float(tau), ctypes.c_float(q_scale), _p(state),
                            ctypes.c_long(stride), _p(out), _p(seq_starts), _p(state_slots), B, nh, dim, vdim, _stream()),
        "gla_scan")
    return out


def gla_chunked(proj: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, z_bias: Optional[torch.Tensor],
                tau: float, q_scale: float, state: torch.Tensor, out: torch.Tensor, seq_starts: torch.Tensor,
                state_slots: torch.Tensor, tiles: torch.Tensor, num_tiles: int, first_request: int, nh: int, dim: int,
                vdim: int, records: Optional[torch.Tensor] = None, decay: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`gla_scan` for the requests that ``tiles`` names (int32 [n, 2] of (request, first row of a tile of
    PREFILL_TILE_ROWS among the request's rows) in any order: every tile of the requests from ``first_request`` on,
    once): the tiles run side by side, first each
    from a zero state, then a walk over every request's tiles leaves each the state before it, then each again from
    that state, writing its rows; the last leaves the request's slot moved on.  ``records`` fp32 [>= n,
    gla_state_floats] and ``decay`` fp32 [>= n, nh dim] are scratch.  The rows of ``z`` that belong to those requests are left
    holding the decays, not the logits."""
    N = proj.shape[0]
    _rows(proj, max(q_col + nh * dim, k_col + nh * dim, v_col + nh * vdim), "gla_chunked rows")
    _need(z.is_cuda and z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1 and z.shape[1] >= nh * dim
          and z.shape[0] == N, "gla_chunked: z fp32 [N, nh dim]")
    _f32(z_bias, nh * dim, "gla_chunked bias")
    _need(out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (N, nh * vdim),
          "gla_chunked: out [N, nh vdim] fp32")
    _dev(seq_starts, state_slots, tiles)
    _need(seq_starts.dtype == torch.int32 and state_slots.dtype == torch.int32 and tiles.dtype == torch.int32
          and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles, "gla_chunked: int32 starts, slots and tiles")
    floats = gla_state_floats(nh, dim, vdim)
    stride = _state_rows(state, floats, "gla_chunked")
    if records is None:
        records = torch.empty((max(num_tiles, 1), floats), dtype=torch.float32, device=out.device)
    if decay is None:
        decay = torch.empty((max(num_tiles, 1), nh * dim), dtype=torch.float32, device=out.device)
    _need(records.dtype == torch.float32 and records.is_contiguous() and records.numel() >= num_tiles * floats
          and decay.dtype == torch.float32 and decay.is_contiguous() and decay.numel() >= num_tiles * nh * dim,
          "gla_chunked: scratch for every tile")
    _ok(_core().ia_gla_chunked(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), q_col, k_col, v_col, _p(z),
                               int(z.stride(0)), _p(z_bias), ctypes.c_float(tau), ctypes.c_float(q_scale), _p(state),
                               ctypes.c_long(stride), _p(out), _p(seq_starts), _p(state_slots), _p(tiles), int(num_tiles),
                               int(first_request), int(N), _p(records), ctypes.c_long(floats), _p(decay), nh, dim, vdim, _stream()), "gla_chunked")
    return out


def head_norm_gate(o: torch.Tensor, gate: Optional[torch.Tensor], gate_col: int, w: torch.Tensor, eps: float, nh: int,
                   vdim: int, out: torch.Tensor) -> torch.Tensor:
    """out = o / sqrt(mean(o^2) + eps) * w * silu(gate) with the mean over each head's vdim values: o fp32 [N, nh vdim],
    w fp32 [vdim] shared by the heads, gate rows holding nh vdim values from gate_col on."""
    N = o.shape[0]
    _need(o.is_cuda and o.dtype == torch.float32 and o.is_contiguous() and tuple(o.shape) == (N, nh * vdim),
          "head_norm_gate: o [N, nh vdim] fp32")
    _f32(w, vdim, "head_norm_gate weight")
    _need(out.is_cuda and out.is_contiguous() and tuple(out.shape) == (N, nh * vdim) and out.dtype in DTYPE_CODE,
          "head_norm_gate: out [N, nh vdim]")
    if gate is not None:           # without a gate: the norm and the weight alone
        _rows(gate, gate_col + nh * vdim, "head_norm_gate gate")
        _need(out.dtype == gate.dtype and gate.shape[0] == N, "head_norm_gate: out of the gate's dtype")
    _ok(_core().ia_head_norm_gate(_p(o), _p(gate), DTYPE_CODE[out.dtype], int(gate.stride(0)) if gate is not None else 0,
                                  gate_col, _p(w), _p(out), N, nh, vdim, ctypes.c_float(eps), _stream()), "head_norm_gate")
    return out


# ------------------------------------------------------------ the recurrence with given decays (k = 1 - f)
def hgrn2_gates(proj: torch.Tensor, q_col: int, z: torch.Tensor, bias: Optional[torch.Tensor],
                lower: Optional[torch.Tensor], k: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In place: the ``z.shape[1]`` values of every row of ``proj`` from ``q_col`` on become silu of themselves, and
    ``z`` (fp32 [N, C], logits) becomes f = lower + (1 - lower) sigmoid(z + bias).  Returns ``k`` (fp32, like z):
    1 - f, made as (1 - lower) sigmoid(-(z + bias))."""
    N, C = z.shape
    if k is None:
        k = torch.empty_like(z)
    _need(k.is_cuda and k.dtype == torch.float32 and k.shape == z.shape and k.stride() == z.stride(), "hgrn2_gates: k like z")
    _rows(proj, q_col + C, "hgrn2_gates rows")
    _need(z.is_cuda and z.dtype == torch.float32 and z.stride(1) == 1 and proj.shape[0] == N, "hgrn2_gates: z fp32 [N, C]")
    _f32(bias, C, "hgrn2_gates bias")
    _f32(lower, C, "hgrn2_gates lower")
    _ok(_core().ia_hgrn2_gates(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), q_col, _p(z), _p(k), int(z.stride(0)),
                               _p(bias), _p(lower), N, C, _stream()), "hgrn2_gates")
    return k


def hgrn2_scan(proj: torch.Tensor, q_col: int, v_col: int, f: torch.Tensor, k: torch.Tensor, state: torch.Tensor,
               out: torch.Tensor, seq_starts: torch.Tensor, state_slots: torch.Tensor, nh: int, dim: int,
               vdim: int) -> torch.Tensor:
    """:func:`gla_scan` with the decays (``f`` fp32 [N, nh dim]) and the keys (``k`` = 1 - f, like f) given, no factor
    on the queries."""
    _need(k.is_cuda and k.dtype == torch.float32 and k.shape == f.shape and k.stride() == f.stride(), "hgrn2_scan: k like f")
    N, B = proj.shape[0], state_slots.numel()
    _rows(proj, max(q_col + nh * dim, v_col + nh * vdim), "hgrn2_scan rows")
    _need(f.is_cuda and f.dtype == torch.float32 and f.dim() == 2 and f.stride(1) == 1 and f.shape[1] >= nh * dim
          and f.shape[0] == N, "hgrn2_scan: f fp32 [N, nh dim]")
    _need(out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (N, nh * vdim),
          "hgrn2_scan: out [N, nh vdim] fp32")
    _i32(seq_starts, B + 1, "hgrn2_scan seq_starts")
    _i32(state_slots, B, "hgrn2_scan state_slots")
    stride = _state_rows(state, gla_state_floats(nh, dim, vdim), "hgrn2_scan")
    _ok(_core().ia_hgrn2_scan(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), q_col, v_col, _p(f), _p(k), int(f.stride(0)),
                              _p(state), ctypes.c_long(stride), _p(out), _p(seq_starts), _p(state_slots), B, nh, dim, vdim,
                              _stream()), "hgrn2_scan")
    return out


def hgrn2_chunked(proj: torch.Tensor, q_col: int, v_col: int, f: torch.Tensor, k: torch.Tensor, state: torch.Tensor,
                  out: torch.Tensor, seq_starts: torch.Tensor, state_slots: torch.Tensor, tiles: torch.Tensor,
                  num_tiles: int, first_request: int, nh: int, dim: int, vdim: int) -> torch.Tensor:
    """:func:`gla_chunked` with the decays and the keys given (see :func:`hgrn2_scan`)."""
    _need(k.is_cuda and k.dtype == torch.float32 and k.shape == f.shape and k.stride() == f.stride(), "hgrn2_chunked: k like f")
    N = proj.shape[0]
    _rows(proj, max(q_col + nh * dim, v_col + nh * vdim), "hgrn2_chunked rows")
    _need(f.is_cuda and f.dtype == torch.float32 and f.dim() == 2 and f.stride(1) == 1 and f.shape[1] >= nh * dim
          and f.shape[0] == N, "hgrn2_chunked: f fp32 [N, nh dim]")
    _need(out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (N, nh * vdim),
          "hgrn2_chunked: out [N, nh vdim] fp32")
    _dev(seq_starts, state_slots, tiles)
    _need(seq_starts.dtype == torch.int32 and state_slots.dtype == torch.int32 and tiles.dtype == torch.int32
          and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles, "hgrn2_chunked: int32 starts, slots and tiles")
    floats = gla_state_floats(nh, dim, vdim)
    stride = _state_rows(state, floats, "hgrn2_chunked")
    records = torch.empty((max(num_tiles, 1), floats), dtype=torch.float32, device=out.device)
    decay = torch.empty((max(num_tiles, 1), nh * dim), dtype=torch.float32, device=out.device)
    _ok(_core().ia_hgrn2_chunked(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), q_col, v_col, _p(f), _p(k),
                                 int(f.stride(0)), _p(state), ctypes.c_long(stride), _p(out), _p(seq_starts),
                                 _p(state_slots), _p(tiles), int(num_tiles), int(first_request), int(N), _p(records),
                                 ctypes.c_long(floats), _p(decay), nh, dim, vdim, _stream()), "hgrn2_chunked")
    return out


# ------------------------------------------------ attention over a window of keys and pooled blocks before it
WPA_MAX_HEAD_DIM = 640


def wpa_pool_entries(page_size: int, pool: int) -> int:
    """Pooled blocks a page of ``page_size`` positions can hold: those whose last position lies in the page."""
    return (page_size - 1) // pool + 1


def wpa_prepare(proj: torch.Tensor, bias: Optional[torch.Tensor], q_out: torch.Tensor, positions: torch.Tensor,
                slots: torch.Tensor, freq: Optional[torch.Tensor], rot: int, unit_norm: bool, eps: float,
                k_pages: torch.Tensor, v_pages: torch.Tensor, nh: int, nkv: int, d: int, dv: int) -> torch.Tensor:
    """From rows [nh q heads of d | nkv k heads of d | nkv v heads of dv] (+ ``bias`` fp32): rotation of the first
    ``rot`` values of every q and k head (value i with i + rot/2), then (``unit_norm``) every q and k head divided by
    its root mean square; queries to ``q_out`` [N, nh d], keys to ``k_pages`` [pages, nkv, page, d] and values to
    ``v_pages`` (transposed within a page: [pages, nkv, dv, page]) at ``slots``."""
    N = proj.shape[0]
    row = (nh + nkv) * d + nkv * dv
    _rows(proj, row, "wpa_prepare rows")
    _rows(q_out, nh * d, "wpa_prepare q_out")
    _need(q_out.dtype == proj.dtype and q_out.shape[0] == N and proj.dtype in DTYPE_CODE, "wpa_prepare: one dtype")
    _f32(bias, row, "wpa_prepare bias")
    _i32(positions, N, "wpa_prepare positions")
    _i32(slots, N, "wpa_prepare slots")
    if rot:
        _need(freq is not None and freq.is_cuda and freq.dtype in (torch.float32, torch.float64)
              and freq.numel() == rot // 2 and rot % 2 == 0 and rot <= d, "wpa_prepare: rot/2 frequencies, rot even, <= d")
    num_pages, ps = k_pages.shape[0], k_pages.shape[2]
    _need(k_pages.dtype == proj.dtype and v_pages.dtype == proj.dtype and k_pages.is_contiguous() and v_pages.is_contiguous()
          and tuple(k_pages.shape) == (num_pages, nkv, ps, d) and tuple(v_pages.shape) == (num_pages, nkv, dv, ps),
          "wpa_prepare: key pages [num_pages, nkv, page_size, d], value pages [num_pages, nkv, dv, page_size]")
    _ok(_core().ia_wpa_prepare(_p(proj), int(proj.stride(0)), _p(bias), _p(q_out), int(q_out.stride(0)),
                               DTYPE_CODE[proj.dtype], _p(positions), _p(slots), _p(freq if rot else None),
                               1 if (rot and freq.dtype == torch.float64) else 0, int(rot), int(bool(unit_norm)),
                               ctypes.c_float(eps), _p(k_pages), _p(v_pages), N, nh, nkv, d, dv, ps, num_pages, _stream()),
        "wpa_prepare")
    return q_out


def wpa_pool(k_pages: torch.Tensor, v_pages: torch.Tensor, pk_pages: torch.Tensor, pv_pages: torch.Tensor,
             token_seq: torch.Tensor, positions: torch.Tensor, bt_tokens: torch.Tensor, bt_pool: torch.Tensor,
             pool: int) -> None:
    """For every token of the step that is the last of a block of ``pool`` positions: the means of the block's keys
    and values, read from the token pages, into the pooled pages ([pages, nkv, wpa_pool_entries, d | dv])."""
    N = positions.numel()
    num_pages, nkv, ps, d = k_pages.shape
    dv = v_pages.shape[2]
    _need(tuple(v_pages.shape) == (num_pages, nkv, dv, ps), "wpa_pool: value pages [num_pages, nkv, dv, page_size]")
    E = wpa_pool_entries(ps, pool)
    _need(tuple(pk_pages.shape[1:]) == (nkv, E, d) and tuple(pv_pages.shape[1:]) == (nkv, E, dv)
          and pk_pages.dtype == k_pages.dtype == v_pages.dtype == pv_pages.dtype and pk_pages.is_contiguous()
          and pv_pages.is_contiguous() and pk_pages.shape[0] == pv_pages.shape[0],
          "wpa_pool: pooled pages [num_pages, nkv, entries, d | dv] of the token pages' dtype")
    _i32(token_seq, N, "wpa_pool token_seq")
    _need(bt_tokens.dtype == torch.int32 and bt_pool.dtype == torch.int32 and bt_tokens.dim() == 2 and bt_pool.dim() == 2
          and bt_tokens.is_contiguous() and bt_pool.is_contiguous(), "wpa_pool: int32 block tables")
    _dev(k_pages, v_pages, pk_pages, pv_pages, token_seq, positions, bt_tokens, bt_pool)
    _ok(_core().ia_wpa_pool(_p(k_pages), _p(v_pages), _p(pk_pages), _p(pv_pages), DTYPE_CODE[k_pages.dtype], _p(token_seq),
                            _p(positions), _p(bt_tokens), bt_tokens.shape[1], _p(bt_pool), bt_pool.shape[1], N, nkv, d, dv,
                            ps, num_pages, pk_pages.shape[0], int(pool), _stream()), "wpa_pool")


def wpa_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, pk_pages: Optional[torch.Tensor],
                  pv_pages: Optional[torch.Tensor], out: torch.Tensor, sinks: Optional[torch.Tensor],
                  token_seq: torch.Tensor, positions: torch.Tensor, bt_tokens: torch.Tensor,
                  bt_pool: Optional[torch.Tensor], nh: int, nkv: int, scale: float, window: int, pool: int) -> torch.Tensor:
    """A query at position p sees keys p - window + 1 .. p (``window`` 0: all from 0) and, with ``pool`` > 0, every
    block of ``pool`` positions that ends at or before p - window, through the means in the pooled pages; one softmax
    over both, ``sinks`` fp32 [nh] in its denominator.  ``out`` [N, nh dv]."""
    N = out.shape[0]
    num_pages, _, ps, d = k_pages.shape
    dv = v_pages.shape[2]
    _rows(q, nh * d, "wpa_attention q")
    _need(out.is_cuda and out.is_contiguous() and tuple(out.shape) == (N, nh * dv) and q.shape[0] == N
          and q.dtype == out.dtype == k_pages.dtype == v_pages.dtype and q.dtype in DTYPE_CODE
          and tuple(k_pages.shape) == (num_pages, nkv, ps, d) and tuple(v_pages.shape) == (num_pages, nkv, dv, ps)
          and k_pages.is_contiguous() and v_pages.is_contiguous(), "wpa_attention: q, pages and out [N, nh dv] of one dtype")
    _f32(sinks, nh, "wpa_attention sinks")
    _i32(token_seq, N, "wpa_attention token_seq")
    _i32(positions, N, "wpa_attention positions")
    _need(bt_tokens.dtype == torch.int32 and bt_tokens.dim() == 2 and bt_tokens.is_contiguous(), "wpa_attention: block tables")
    pooled = pool > 0 and window > 0
    if pooled:
        _need(pk_pages is not None and pv_pages is not None and bt_pool is not None and bt_pool.dtype == torch.int32
              and bt_pool.is_contiguous() and pk_pages.dtype == q.dtype and pv_pages.dtype == q.dtype
              and tuple(pk_pages.shape[1:]) == (nkv, wpa_pool_entries(ps, pool), d)
              and tuple(pv_pages.shape[1:]) == (nkv, wpa_pool_entries(ps, pool), dv), "wpa_attention: pooled pages")
    _dev(q, k_pages, v_pages, pk_pages, pv_pages, out, token_seq, positions, bt_tokens, bt_pool)
    _ok(_core().ia_wpa_attention(_p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(pk_pages if pooled else None),
                                 _p(pv_pages if pooled else None), _p(out), nh * dv, DTYPE_CODE[out.dtype], _p(sinks),
                                 _p(token_seq), _p(positions), _p(bt_tokens), bt_tokens.shape[1],
                                 _p(bt_pool if pooled else None), bt_pool.shape[1] if pooled else 0, N, nh, nkv, d, dv, ps,
                                 num_pages, pk_pages.shape[0] if pooled else 0, ctypes.c_float(scale), int(window),
                                 int(pool) if pooled else 0, _stream()), "wpa_attention")
    return out


def wpa_mfma_available(d: int, dv: int) -> bool:
    """Whether the matrix-core kernels of the window-and-blocks attention take these key and value sizes (their
    library is built at its first use)."""
    return d in _build.SUPPORTED_HEAD_DIMS and dv in _build.SUPPORTED_HEAD_DIMS


def _wpa(d: int, dv: int) -> ctypes.CDLL:
    return load_library(f"wpa_d{d}_v{dv}")


def _wpa_check(q, k_pages, v_pages, pk_pages, pv_pages, out, sinks, bt_tokens, bt_pool, nh, nkv, window, pool, what):
    num_pages, _, ps, d = k_pages.shape
    dv = v_pages.shape[2]
    N = out.shape[0]
    _rows(q, nh * d, f"{what} q")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16
          and v_pages.dtype == torch.bfloat16 and out.is_cuda and out.is_contiguous() and tuple(out.shape) == (N, nh * dv)
          and tuple(k_pages.shape) == (num_pages, nkv, ps, d) and tuple(v_pages.shape) == (num_pages, nkv, dv, ps)
          and k_pages.is_contiguous() and v_pages.is_contiguous() and ps % 4 == 0 and q.stride(0) % 8 == 0,
          f"{what}: bf16 q, key pages [num_pages, nkv, page_size, d], value pages [num_pages, nkv, dv, page_size] with "
          "a page size in fours, out [N, nh dv]")
    _f32(sinks, nh, f"{what} sinks")
    _need(bt_tokens.dtype == torch.int32 and bt_tokens.dim() == 2 and bt_tokens.is_contiguous(), f"{what}: block tables")
    pooled = pool > 0 and window > 0
    if pooled:
        E = wpa_pool_entries(ps, pool)
        _need(pk_pages is not None and pv_pages is not None and bt_pool is not None and bt_pool.dtype == torch.int32
              and bt_pool.is_contiguous() and pk_pages.dtype == q.dtype and pv_pages.dtype == q.dtype
              and pk_pages.is_contiguous() and pv_pages.is_contiguous()
              and tuple(pk_pages.shape[1:]) == (nkv, E, d) and tuple(pv_pages.shape[1:]) == (nkv, E, dv), f"{what}: pooled pages")
    _dev(q, k_pages, v_pages, pk_pages, pv_pages, out, bt_tokens, bt_pool)
    return pooled, ps, num_pages, d, dv


def wpa_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, pk_pages: Optional[torch.Tensor],
               pv_pages: Optional[torch.Tensor], out: torch.Tensor, sinks: Optional[torch.Tensor],
               positions: torch.Tensor, bt_tokens: torch.Tensor, bt_pool: Optional[torch.Tensor], nh: int, nkv: int,
               scale: float, window: int, pool: int) -> torch.Tensor:
    """:func:`wpa_attention` of B single tokens on the matrix cores, bf16: row b of q, out and the block tables is
    token b at positions[b]."""
    pooled, ps, num_pages, d, dv = _wpa_check(q, k_pages, v_pages, pk_pages, pv_pages, out, sinks, bt_tokens, bt_pool,
                                              nh, nkv, window, pool, "wpa_decode")
    B = out.shape[0]
    _i32(positions, B, "wpa_decode positions")
    _need(bt_tokens.shape[0] >= B and (not pooled or bt_pool.shape[0] >= B), "wpa_decode: a row of the block tables a token")
    _ok(_wpa(d, dv).ia_wpa_decode(_p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(pk_pages if pooled else None),
                                  _p(pv_pages if pooled else None), _p(out), _p(sinks), _p(positions), _p(bt_tokens),
                                  bt_tokens.shape[1], _p(bt_pool if pooled else None), bt_pool.shape[1] if pooled else 0,
                                  B, nh, nkv, ps, num_pages, pk_pages.shape[0] if pooled else 0, ctypes.c_float(scale),
                                  int(window), int(pool) if pooled else 0, _stream()), "wpa_decode")
    return out


def wpa_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, pk_pages: Optional[torch.Tensor],
                pv_pages: Optional[torch.Tensor], out: torch.Tensor, sinks: Optional[torch.Tensor],
                seq_starts: torch.Tensor, seq_ctx: torch.Tensor, bt_tokens: torch.Tensor, bt_pool: Optional[torch.Tensor],
                tiles: torch.Tensor, num_tiles: int, nh: int, nkv: int, scale: float, window: int, pool: int) -> torch.Tensor:
    """:func:`wpa_attention` of portions of prompts on the matrix cores, bf16: request s brings rows seq_starts[s] ..
    seq_starts[s+1]-1 after seq_ctx[s] cached tokens; tiles[i] = (s, first row of a block of PREFILL_TILE_ROWS)."""
    pooled, ps, num_pages, d, dv = _wpa_check(q, k_pages, v_pages, pk_pages, pv_pages, out, sinks, bt_tokens, bt_pool,
                                              nh, nkv, window, pool, "wpa_prefill")
    B = bt_tokens.shape[0]
    _i32(seq_starts, B + 1, "wpa_prefill seq_starts")
    _i32(seq_ctx, B, "wpa_prefill seq_ctx")
    _need(tiles.dtype == torch.int32 and tiles.is_cuda and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles,
          "wpa_prefill: tiles int32 [num_tiles, 2]")
    _ok(_wpa(d, dv).ia_wpa_prefill(_p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(pk_pages if pooled else None),
                                   _p(pv_pages if pooled else None), _p(out), _p(sinks), _p(seq_starts), _p(seq_ctx),
                                   _p(bt_tokens), bt_tokens.shape[1], _p(bt_pool if pooled else None),
                                   bt_pool.shape[1] if pooled else 0, _p(tiles), int(num_tiles), nh, nkv, ps, num_pages,
                                   pk_pages.shape[0] if pooled else 0, ctypes.c_float(scale), int(window),
                                   int(pool) if pooled else 0, _stream()), "wpa_prefill")
    return out


def rms_rows(x: torch.Tensor, col: int, cols: int, weight: Optional[torch.Tensor], eps: float,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n] = x[n, col : col + cols] / sqrt(mean of its squares + eps) * weight, in x's dtype."""
    _rows(x, col + cols, "rms_rows x")
    N = x.shape[0]
    if out is None:
        out = torch.empty((N, cols), dtype=x.dtype, device=x.device)
    _need(out.is_cuda and out.dtype == x.dtype and tuple(out.shape) == (N, cols) and out.is_contiguous(), "rms_rows: out [N, cols]")
    if weight is not None:
        _need(weight.is_cuda and weight.dtype in DTYPE_CODE and weight.numel() == cols and weight.is_contiguous(),
              "rms_rows: a weight a column")
    _ok(_core().ia_rms_rows(ctypes.c_void_p(x.data_ptr() + col * x.element_size()), int(x.stride(0)), _p(weight),
                            DTYPE_CODE[weight.dtype] if weight is not None else 0, _p(out), cols, DTYPE_CODE[x.dtype], N,
                            cols, ctypes.c_float(eps), _stream()), "rms_rows")
    return out


def gelu_mul_rows(u: torch.Tensor, table: torch.Tensor, col: int, ids: torch.Tensor,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[n, j] = gelu_tanh(u[n, j]) * table[ids[n], col + j]."""
    N, C = u.shape
    _need(u.is_cuda and u.is_contiguous() and u.dtype in DTYPE_CODE, "gelu_mul_rows: u [N, C]")
    _need(table.is_cuda and table.dim() == 2 and table.is_contiguous() and table.dtype in DTYPE_CODE
          and 0 <= col and col + C <= table.shape[1], "gelu_mul_rows: the table's rows are too short")
    _i32(ids, N, "gelu_mul_rows ids")
    if out is None:
        out = torch.empty_like(u)
    _need(out.is_cuda and out.is_contiguous() and out.dtype == u.dtype and out.shape == u.shape, "gelu_mul_rows: out like u")
    _ok(_core().ia_gelu_mul_rows(_p(u), _p(out), DTYPE_CODE[u.dtype], _p(table), DTYPE_CODE[table.dtype], table.shape[1],
                                 int(col), _p(ids), table.shape[0], N, C, _stream()), "gelu_mul_rows")
    return out


def sigattn_prepare(proj: torch.Tensor, bq, bk, bv, wq: torch.Tensor, wk: Optional[torch.Tensor], eps: float,
                    temp_coef: float, temp_every: int, positions: torch.Tensor, slots: Optional[torch.Tensor],
                    q_out: torch.Tensor, k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], nh: int,
                    nkv: int, dim: int, vdim: int) -> torch.Tensor:
    """From rows [q: nh dim | k: nkv dim | v: nkv vdim | ...]: biases, the norm over all of a row's queries (keys)
    with weights wq (wk), the queries' factor 1 + temp_coef ln(floor((p + 1) / temp_every) + 1) (temp_every 0: none);
    queries to ``q_out`` [N, nh dim], keys and values to their pages at ``slots`` (None: queries only)."""
    N = proj.shape[0]
    _rows(proj, nh * dim + (nkv * (dim + vdim) if slots is not None else 0), "sigattn_prepare rows")
    _f32(bq, nh * dim, "sigattn_prepare bq"); _f32(bk, nkv * dim, "sigattn_prepare bk"); _f32(bv, nkv * vdim, "sigattn_prepare bv")
    _f32(wq, nh * dim, "sigattn_prepare wq"); _f32(wk, nkv * dim, "sigattn_prepare wk")
    _need(q_out.is_cuda and q_out.is_contiguous() and tuple(q_out.shape) == (N, nh * dim) and q_out.dtype == proj.dtype,
          "sigattn_prepare: q_out [N, nh dim] of the rows' dtype")
    _i32(positions, N, "sigattn_prepare positions")
    ps = num_pages = 0
    if slots is not None:
        _i32(slots, N, "sigattn_prepare slots")
        _dev(k_pages, v_pages)
        num_pages, ps = k_pages.shape[0], k_pages.shape[2]
        _need(tuple(k_pages.shape) == (num_pages, nkv, ps, dim) and tuple(v_pages.shape) == (num_pages, nkv, vdim, ps)
              and k_pages.dtype == proj.dtype and v_pages.dtype == proj.dtype,
              "sigattn_prepare: pages [P, nkv, page, dim] and [P, nkv, vdim, page] of the rows' dtype")
    _ok(_core().ia_sigattn_prepare(_p(proj), DTYPE_CODE[proj.dtype], int(proj.stride(0)), _p(bq), _p(bk), _p(bv), _p(wq),
                                   _p(wk), ctypes.c_float(eps), ctypes.c_float(temp_coef), int(temp_every),
                                   _p(positions), _p(slots), _p(q_out), _p(k_pages), _p(v_pages), N, nh, nkv, dim, vdim,
                                   ps, num_pages, _stream()), "sigattn_prepare")
    return q_out


def _check_sigattn(q, k_pages, v_pages, gate, out, nh, nkv, dim, vdim, what):
    N = q.shape[0]
    _rows(q, nh * dim, what + " queries")
    _dev(k_pages, v_pages, out)
    num_pages, ps = k_pages.shape[0], k_pages.shape[2]
    _need(tuple(k_pages.shape) == (num_pages, nkv, ps, dim) and tuple(v_pages.shape) == (num_pages, nkv, vdim, ps)
          and k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, what + ": pages of the queries' dtype and sizes")
    _need(tuple(out.shape) == (N, nh * vdim) and out.dtype == q.dtype, what + ": out [N, nh vdim]")
    if gate is not None:
        _rows(gate, nh, what + " gate")
        _need(gate.dtype == q.dtype and gate.shape[0] == N, what + ": a gate row per query row")
    return N, num_pages, ps


def sigattn_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, gate: Optional[torch.Tensor],
                    out: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor,
                    r1, r2, pb, nh: int, nkv: int, dim: int, vdim: int, scale: float) -> torch.Tensor:
    """out[n, h] = sigmoid(gate[n, h]) sum_{j <= p} sigmoid(scale q.k_j - r1_h ln(1 + r2_h (p - j)) + pb_h) v_j, the
    plain kernel (one wave per token and head, fp32 arithmetic)."""
    N, num_pages, ps = _check_sigattn(q, k_pages, v_pages, gate, out, nh, nkv, dim, vdim, "sigattn_generic")
    for t in (r1, r2, pb):
        _f32(t, nh, "sigattn_generic per-head numbers")
    _i32(token_seq, N, "sigattn token_seq"); _i32(positions, N, "sigattn positions")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(), "sigattn: block tables")
    _ok(_core().ia_sigattn_generic(_p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(gate),
                                   int(gate.stride(0)) if gate is not None else 0, _p(out), DTYPE_CODE[q.dtype],
                                   _p(token_seq), _p(positions), _p(block_tables), block_tables.shape[1], _p(r1), _p(r2),
                                   _p(pb), N, nh, nkv, dim, vdim, ps, num_pages, ctypes.c_float(scale), _stream()),
        "sigattn_generic")
    return out


def sigattn_mfma_available(dim: int, vdim: int) -> bool:
    """Whether the matrix-core kernels of the sigmoid attention take these key and value sizes (their library is
    built at its first use)."""
    return dim in _build.SUPPORTED_HEAD_DIMS and vdim in _build.SUPPORTED_HEAD_DIMS


def _sigattn(dim: int, vdim: int) -> ctypes.CDLL:
    return load_library(f"sigattn_d{dim}_v{vdim}")


def sigattn_decode_parts(batch: int, nh: int, nkv: int, max_len: int, device: Optional[torch.device] = None) -> int:
    """Parts the keys of a single token are cut into by :func:`sigattn_decode`: enough workgroups (one per token,
    group of up to 16 heads of a key/value head, and part) for about two a compute unit, no part shorter than the 64
    keys that a workgroup's four waves take at a time, at most 64 parts."""
    groups = batch * nkv * (-(-(nh // nkv) // 16))
    wanted = -(-2 * compute_units(device) // max(groups, 1))
    return max(1, min(wanted, -(-max_len // 64), 64))


def sigattn_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, gate: Optional[torch.Tensor],
                   out: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor, r1, r2, pb, nh: int, nkv: int,
                   dim: int, vdim: int, scale: float, max_len: int, parts: Optional[int] = None) -> torch.Tensor:
    """:func:`sigattn_generic` for B single tokens (row b: token b at positions[b], row b of the block tables) in bf16
    on the matrix cores.  ``max_len`` bounds the positions (host side) and sets into how many parts the keys are cut."""
    B, num_pages, ps = _check_sigattn(q, k_pages, v_pages, gate, out, nh, nkv, dim, vdim, "sigattn_decode")
    _need(q.dtype == torch.bfloat16 and ps % 4 == 0, "sigattn_decode: bf16, and a page size that is a multiple of 4")
    for t in (r1, r2, pb):
        _f32(t, nh, "sigattn_decode per-head numbers")
    _i32(positions, B, "sigattn_decode positions")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
          and block_tables.shape[0] >= B and block_tables.shape[1] * ps >= max_len, "sigattn_decode: block tables")
    parts = parts or sigattn_decode_parts(B, nh, nkv, max_len, out.device)
    part = torch.empty(B * parts * nh * vdim, dtype=torch.float32, device=out.device) if parts > 1 else None
    _ok(_sigattn(dim, vdim).ia_sigattn_decode(
        _p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(gate), int(gate.stride(0)) if gate is not None else 0,
        _p(out), _p(part), _p(positions), _p(block_tables), block_tables.shape[1], _p(r1), _p(r2), _p(pb), B, nh, nkv, ps,
        num_pages, ctypes.c_float(scale), int(parts), _stream()), "sigattn_decode")
    return out


def sigattn_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, gate: Optional[torch.Tensor],
                    out: torch.Tensor, seq_starts: torch.Tensor, seq_ctx: torch.Tensor, block_tables: torch.Tensor,
                    tiles: torch.Tensor, num_tiles: int, r1, r2, pb, nh: int, nkv: int, dim: int, vdim: int,
                    scale: float) -> torch.Tensor:
    """:func:`sigattn_generic` for portions of prompts in bf16 on the matrix cores: request s has the rows
    seq_starts[s] .. seq_starts[s + 1] - 1, seq_ctx[s] keys before them and row s of the block tables; tiles[i] =
    (s, first row of a block of PREFILL_TILE_ROWS among the request's rows).  Rows of no tile are left alone."""
    N, num_pages, ps = _check_sigattn(q, k_pages, v_pages, gate, out, nh, nkv, dim, vdim, "sigattn_prefill")
    _need(q.dtype == torch.bfloat16 and ps % 4 == 0, "sigattn_prefill: bf16, and a page size that is a multiple of 4")
    for t in (r1, r2, pb):
        _f32(t, nh, "sigattn_prefill per-head numbers")
    _dev(seq_starts, seq_ctx, tiles)
    _need(seq_starts.dtype == torch.int32 and seq_ctx.dtype == torch.int32 and tiles.dtype == torch.int32
          and tiles.is_contiguous() and tiles.numel() >= 2 * num_tiles, "sigattn_prefill: int32 starts, contexts and tiles")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(), "sigattn_prefill: block tables")
    _ok(_sigattn(dim, vdim).ia_sigattn_prefill(
        _p(q), int(q.stride(0)), _p(k_pages), _p(v_pages), _p(gate), int(gate.stride(0)) if gate is not None else 0,
        _p(out), _p(seq_starts), _p(seq_ctx), _p(block_tables), block_tables.shape[1], _p(tiles), int(num_tiles), _p(r1),
        _p(r2), _p(pb), nh, nkv, ps, num_pages, ctypes.c_float(scale), _stream()), "sigattn_prefill")
    return out


# ------------------------------------------------------------------------- sampling
def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "argmax: logits must be fp32")
    _i32(out, R, "argmax out")
    _ok(_core().ia_argmax(_p(logits), V, _p(out), R, V, _stream()), "argmax")
    return out


def repetition_penalty(logits: torch.Tensor, recent: torch.Tensor, counts: torch.Tensor,
                       penalty: torch.Tensor, previous: Optional[torch.Tensor] = None,
                       previous_index: Optional[torch.Tensor] = None) -> None:
    """Every token of recent[r, :counts[r]] is penalised in row r (a positive logit divided by penalty[r], another
    multiplied by it; a token that stands twice, twice).  ``previous`` (int32 tokens that an earlier launch left
    on the device) and ``previous_index`` (int32 [R]: which of them is row r's newest token, -1: none) add a token
    that the host has not seen yet."""
    _dev(logits, recent, counts, penalty, previous, previous_index)
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "penalty: logits must be fp32")
    _need(recent.dtype == torch.int32 and recent.dim() == 2 and recent.shape[0] == R, "penalty: recent int32 [R, W]")
    _i32(counts, R, "penalty counts")
    _need(penalty.dtype == torch.float32 and penalty.numel() == R, "penalty: one fp32 factor per row")
    if previous is not None or previous_index is not None:
        _need(previous is not None and previous_index is not None and previous.dtype == torch.int32
              and previous.is_contiguous(), "penalty: previous tokens int32 with their index")
        _i32(previous_index, R, "penalty previous_index")
    _ok(_core().ia_repetition_penalty(_p(logits), V, _p(recent), recent.shape[1], _p(counts), _p(penalty),
                                      _p(previous), _p(previous_index), R, V, _stream()), "repetition_penalty")


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           u: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _dev(logits, work, temperature, top_p, u, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and work.dtype == torch.float32 and work.numel() >= R * V,
          "sample: logits fp32 [R, V] and fp32 work space of the same size")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        _need(t.dtype == torch.float32 and t.numel() == R, f"sample: {name} must hold one fp32 value per row")
    _i32(out, R, "sample out")
    _ok(_core().ia_sample(_p(logits), V, _p(work), _p(temperature), _p(top_p), _p(u), _p(out), R, V, _stream()),
        "sample")
    return out


# ---------------------------------------------------- which head sizes the MFMA kernels take
def attention_mfma_available(d: int) -> bool:
    """Whether the MFMA attention kernels take head size d (their library is built at its first use)."""
    return d in _build.SUPPORTED_HEAD_DIMS


# ------------------------------------------------- time per kernel, by the device's clock
# INFERNUM_PROFILE=1 in the environment (or ``set_profile(True)``): every call of a kernel function of this
# module is bracketed by two events on its stream, and a table of calls and device time per function goes to
# standard error when the process ends (``profile_report`` gives it at any time).  The reference's switch of the
# same name prints the time per operation of its graph executor (infernum-cpu/src/executor.rs:24-71).  Steps
# are not recorded into HIP graphs meanwhile (a replayed launch has no call to bracket).
_PROFILED = ("sigattn_decode", "sigattn_prefill", "gemm_mfma_grouped", "norm_add", "activation", "latent_prepare", "gemm_heads", "router_topk", "moe_experts", "cast", "copy_pages", "gather_tokens", "words_from_host", "words_to_host", "embed", "add_rmsnorm", "residual_add", "rope_kv_append", "swiglu", "gemm_generic", "gemm_mfma",
             "gemm_library", "gemm_skinny", "gemm_skinny_rows", "attention_generic", "attention_decode", "attention_decode_rotating",
             "attention_prefill", "argmax", "repetition_penalty", "sample")
_profile_on = False
_profile_open: List[Tuple[str, "torch.cuda.Event", "torch.cuda.Event"]] = []
_profile_sum: Dict[str, List[float]] = {}          # function -> [calls, milliseconds]
_plain = {name: globals()[name] for name in _PROFILED}


def _fold_profile() -> None:
    if _profile_open:
        torch.cuda.synchronize()
        for name, a, b in _profile_open:
            acc = _profile_sum.setdefault(name, [0, 0.0])
            acc[0] += 1
            acc[1] += a.elapsed_time(b)
        _profile_open.clear()


def _timed(name: str, fn):
    @functools.wraps(fn)
    def call(*args, **kw):
        if not _profile_on or torch.cuda.is_current_stream_capturing():
            return fn(*args, **kw)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        try:
            return fn(*args, **kw)
        finally:
            b.record()
            _profile_open.append((name, a, b))
            if len(_profile_open) >= 4096:
                _fold_profile()
    return call


for _name in _PROFILED:
    globals()[_name] = _timed(_name, _plain[_name])


def profiling() -> bool:
    return _profile_on


def set_profile(on: bool) -> bool:
    """Switch the timing of every kernel call on or off; returns what it was.  Engines made while it is on
    do not record their decode steps into graphs."""
    global _profile_on
    before, _profile_on = _profile_on, bool(on)
    return before


def profile_report(reset: bool = False) -> Dict[str, Tuple[int, float]]:
    """function -> (calls, milliseconds on the device) since the start or the last reset."""
    _fold_profile()
    out = {k: (int(v[0]), float(v[1])) for k, v in _profile_sum.items()}
    if reset:
        _profile_sum.clear()
    return out


def _print_profile() -> None:
    try:
        rep = profile_report()
    except Exception:                                   # the device is gone at exit: nothing to print
        return
    if not rep:
        return
    total = sum(ms for _, ms in rep.values())
    print(f"[infernum_amd profile] {total:.3f} ms in {sum(c for c, _ in rep.values())} kernel calls", file=sys.stderr)
    for name, (calls, ms) in sorted(rep.items(), key=lambda kv: -kv[1][1]):
        print(f"[infernum_amd profile] {name:28s} {calls:8d} calls {ms:12.3f} ms {ms / calls * 1e3:10.1f} us/call "
              f"{100 * ms / total:5.1f} %", file=sys.stderr)


if os.environ.get("INFERNUM_PROFILE") == "1":
    _profile_on = True
atexit.register(_print_profile)
