"""The Sikazen decoder, plainly: whole sequences, no cache, float64, one function per mechanism.

It shares nothing with the package: a model is a configuration (the dict that config.json holds) and a dict of
tensors by their names in a file.  ``round_to=torch.bfloat16`` rounds what a bfloat16 engine stores between its
kernels, which tells how far rounding alone moves the logits.

Notation.  W: the stream's width; x [T, W] the stream; e0 [T, W] the scaled embedding rows.  A layer:

    x <- x + mixer(g1 n(x)) + ff(g2 n(x)),      n(y) = y / sqrt(mean(y^2) + eps),   g1, g2 single numbers
    t = side_table[token][i d : (i + 1) d];  y = P (gelu_tanh(G x) * t);  x <- x + n(y) * w_side

Layers ``start .. stop - 1`` run ``times`` times in a row with the same tensors; before every pass but the first,
x <- x + e0.
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Tuple

import torch

F64 = torch.float64


def _r(x: torch.Tensor, round_to) -> torch.Tensor:
    return x if round_to is None else x.to(round_to).to(F64)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ---------------------------------------------------------------------------------------------- rotation
def rotation_angles(positions: torch.Tensor, dims: int, base: float, factor: float = 1.0) -> torch.Tensor:
    """[T, dims / 2]: position times base^(-2i/dims) / factor."""
    i = torch.arange(dims // 2, dtype=F64)
    freq = base ** (-2.0 * i / dims) / factor
    return positions.to(F64)[:, None] * freq[None, :]


def rotate(x: torch.Tensor, angles: torch.Tensor, dims: int, layout: str) -> torch.Tensor:
    """x [T, heads, d]: the first ``dims`` values of every head are rotated, pair by pair.  ``layout`` "half": value i
    with value i + dims/2; "pairs": value 2i with value 2i + 1."""
    out = x.clone()
    cos, sin = torch.cos(angles)[:, None, :], torch.sin(angles)[:, None, :]
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * cos - v * sin
        out[..., dims // 2:dims] = v * cos + u * sin
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------------------------- mixers
def pooled_window_weights(scores: torch.Tensor, pooled_scores: torch.Tensor, size: int, pool: int):
    """One head.  scores [T, T] (query i, key j), pooled_scores [T, B] (query i, block b).  Query i sees key j when
    0 <= i - j < size, and block b when its last position b pool + pool - 1 <= i - size.  One softmax over both.
    Returns the weights (on keys [T, T], on blocks [T, B])."""
    T, B = scores.shape[0], pooled_scores.shape[1]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < size)
    b = torch.arange(B)[None, :]
    seen_b = (b * pool + pool - 1) <= (i - size)
    both = torch.cat([scores.masked_fill(~seen, -math.inf), pooled_scores.masked_fill(~seen_b, -math.inf)], dim=1)
    w = torch.softmax(both, dim=1)
    return w[:, :T], w[:, T:]


def attention_mixer(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                    round_to=None) -> torch.Tensor:
    """Grouped-query attention with biases, rotation of halves, a unit norm of every rotated query and key head, a
    window of single keys and, before it, whole blocks of keys seen through their means."""
    T = a.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _r(a @ w[p + "q"].T + w[p + "q.b"], round_to).view(T, H, d)
    k = _r(a @ w[p + "k"].T + w[p + "k.b"], round_to).view(T, G, d)
    v = _r(a @ w[p + "v"].T + w[p + "v.b"], round_to).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        ang = rotation_angles(torch.arange(T), rot["dims"], float(rot["base"]), factor)
        q, k = rotate(q, ang, rot["dims"], "half"), rotate(k, ang, rot["dims"], "half")
    q, k = _r(unit_rms(q, eps), round_to), _r(unit_rms(k, eps), round_to)
    mask = m.get("mask")
    size = int(mask["size"]) if mask else T + 1                  # no mask: every earlier key
    pool = int(mask["pool"]) if mask and mask.get("pool") else T + 1          # no blocks: what leaves the window is gone
    B = T // pool
    out = torch.zeros((T, H, dv), dtype=F64)
    for h in range(H):
        g = h // (H // G)
        kp = k[: B * pool, g].view(B, pool, d).mean(dim=1)
        vp = v[: B * pool, g].view(B, pool, dv).mean(dim=1)
        kp, vp = _r(kp, round_to), _r(vp, round_to)
        wk, wb = pooled_window_weights(q[:, h] @ k[:, g].T * m["scale"], q[:, h] @ kp.T * m["scale"], size, pool)
        out[:, h] = wk @ v[:, g] + wb @ vp
    return _r(out.reshape(T, H * dv), round_to) @ w[p + "o"].T


def sink_softmax(scores: torch.Tensor, sink: float) -> torch.Tensor:
    """Causal softmax over [T, T] scores whose denominator also holds exp(sink)."""
    T = scores.shape[0]
    s = scores.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -math.inf)
    top = torch.maximum(s.max(dim=1, keepdim=True).values, torch.tensor(sink, dtype=F64))
    ex = torch.exp(s - top)
    return ex / (ex.sum(dim=1, keepdim=True) + torch.exp(sink - top))


def latent_attention_mixer(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                           round_to=None) -> torch.Tensor:
    """Queries through a normed latent; keys and values of all heads from one normed latent a token, plus one
    rotated key part that the heads share; rotation of neighbouring pairs; a sink in every head's softmax."""
    T = a.shape[0]
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = _r(unit_rms(_r(a @ w[p + "dq"].T, round_to), eps) * w[p + "dq.norm"], round_to)
    q = _r(cq @ w[p + "uq"].T, round_to).view(T, H, d + dr)
    lat = _r(a @ w[p + "dkv"].T, round_to)
    c = _r(unit_rms(lat[:, :rank], eps) * w[p + "dkv.norm"], round_to)
    r = lat[:, rank:].view(T, 1, dr)
    rot = m["rot"]
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    ang = rotation_angles(torch.arange(T), rot["dims"], float(rot["base"]), factor)
    q_rot = rotate(q[..., d:].contiguous(), ang, rot["dims"], "pairs")
    r = _r(rotate(r, ang, rot["dims"], "pairs"), round_to)[:, 0]
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    val = (c @ w[p + "uv"].T).view(T, H, dv)
    out = torch.zeros((T, H, dv), dtype=F64)
    for h in range(H):
        s = (q[:, h, :d] @ k_plain[:, h].T + q_rot[:, h] @ r.T) * m["scale"]
        out[:, h] = sink_softmax(s, float(w[p + "sink"][h])) @ val[:, h]
    return _r(out.reshape(T, H * dv), round_to) @ w[p + "o"].T


def hgrn2_gates(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str) -> torch.Tensor:
    """The forget gate per token and channel: lower + (1 - lower) sigmoid(F a + b)."""
    low = w[p + "lower"]
    return low + (1.0 - low) * sigmoid(a @ w[p + "f"].T + w[p + "f.b"])


def hgrn2_recurrence(q: torch.Tensor, f: torch.Tensor, v: torch.Tensor, state: Optional[torch.Tensor] = None):
    """One head, token after token: S <- diag(f_t) S + (1 - f_t) v_t^T, o_t = S^T q_t.  q, f [T, dim], v [T, vdim]."""
    T, dim = q.shape
    S = torch.zeros((dim, v.shape[1]), dtype=F64) if state is None else state.clone()
    out = torch.empty((T, v.shape[1]), dtype=F64)
    for t in range(T):
        S = f[t][:, None] * S + (1.0 - f[t])[:, None] * v[t][None, :]
        out[t] = S.T @ q[t]
    return out, S


def hgrn2_mixer(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float, round_to=None) -> torch.Tensor:
    T = a.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = _r(silu(_r(a @ w[p + "q"].T, round_to)), round_to).view(T, H, d)
    v = _r(a @ w[p + "v"].T, round_to).view(T, H, dv)
    if round_to is not None:
        f = w[p + "lower"] + (1.0 - w[p + "lower"]) * sigmoid(_r(a @ w[p + "f"].T, round_to) + w[p + "f.b"])
    else:
        f = hgrn2_gates(a, w, p)
    f = f.view(T, H, d)
    out = torch.empty((T, H, dv), dtype=F64)
    for h in range(H):
        o, _ = hgrn2_recurrence(q[:, h], f[:, h], v[:, h])
        out[:, h] = unit_rms(o, eps) * w[p + "norm"]
    return _r(out.reshape(T, H * dv), round_to) @ w[p + "o"].T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "hgrn2": hgrn2_mixer}


# ---------------------------------------------------------------------------------------------- the rest
def gated_feed_forward(f: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, round_to=None) -> torch.Tensor:
    act = _r(silu(f @ w[p + "gate"].T) * (f @ w[p + "up"].T), round_to)
    return act @ w[p + "down"].T


def token_side_input(x: torch.Tensor, tokens: torch.Tensor, w: Mapping[str, torch.Tensor], layer: int, dim: int,
                     eps: float, round_to=None) -> torch.Tensor:
    """What layer ``layer`` adds to the stream from its part of the side table's row of every token."""
    p = f"l{layer}.side."
    t = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = _r(gelu_tanh(_r(_r(x, round_to) @ w[p + "gate"].T, round_to)) * t, round_to)
    y = g @ w[p + "proj"].T
    return unit_rms(y, eps) * w[p + "norm"]


def layer_runs(cfg: Mapping) -> List[Tuple[int, bool]]:
    """(layer, whether e0 is added before it) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] <= 1 or loop["stop"] <= loop["start"]:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg: Mapping, w: Mapping[str, torch.Tensor], tokens, round_to=None, streams: Optional[list] = None,
            upto: Optional[int] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``streams``: gets the stream after every layer run.  ``upto``: only
    the first so many layer runs."""
    w = {k: (v.to(F64) if v.dtype.is_floating_point else v) for k, v in w.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])
    e0 = w["embed"][tokens] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    x = e0.clone()
    side = cfg.get("token_side")
    for n, (i, add_e0) in enumerate(layer_runs(cfg)):
        if upto is not None and n >= upto:
            break
        layer = cfg["layers"][i]
        if add_e0:
            x = x + e0
        unit = unit_rms(x, eps)
        a = _r(unit * w[f"l{i}.norm1"], round_to)
        delta = MIXERS[layer["type"]](a, w, f"l{i}.mix.", layer["mixer"], eps, round_to)
        if layer.get("mlp") is not None:
            delta = delta + gated_feed_forward(_r(unit * w[f"l{i}.norm2"], round_to), w, f"l{i}.mlp.", round_to)
        x = x + delta
        if side:
            x = x + token_side_input(x, tokens, w, i, int(side["dim"]), eps, round_to)
        if streams is not None:
            streams.append(x.clone())
    return _r(unit_rms(x, eps) * w["final.norm"], round_to) @ w["head"].T


# ---------------------------------------------------------------------------------------------- weights for tests
def tensor_shapes(cfg: Mapping) -> Dict[str, Tuple[int, ...]]:
    """Names and shapes of a model's tensors."""
    V, W = cfg["vocab"], cfg["width"]
    side = cfg.get("token_side")
    out: Dict[str, Tuple[int, ...]] = {"embed": (V, W)}
    if side:
        out["side.embed"] = (V, int(side["dim"]) * len(cfg["layers"]))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = ()
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, W), p + "mix.q.b": (H * d,), p + "mix.k": (G * d, W), p + "mix.k.b": (G * d,),
                        p + "mix.v": (G * dv, W), p + "mix.v.b": (G * dv,), p + "mix.o": (W, H * dv)})
        elif layer["type"] == "latent_attention":
            H, d, dr, dv, rk, rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (rq, W), p + "mix.dq.norm": (rq,), p + "mix.uq": (H * (d + dr), rq),
                        p + "mix.dkv": (rk + dr, W), p + "mix.dkv.norm": (rk,), p + "mix.uk": (H * d, rk),
                        p + "mix.uv": (H * dv, rk), p + "mix.sink": (H,), p + "mix.o": (W, H * dv)})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, W), p + "mix.f": (H * d, W), p + "mix.f.b": (H * d,),
                        p + "mix.lower": (H * d,), p + "mix.v": (H * dv, W), p + "mix.norm": (dv,), p + "mix.o": (W, H * dv)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (), p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
        if side:
            out.update({p + "side.gate": (int(side["dim"]), W), p + "side.proj": (W, int(side["dim"])), p + "side.norm": (W,)})
    out["final.norm"] = ()
    out["head"] = (V, W)
    return out


def random_weights(cfg: Mapping, seed: int = 0, store: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Weights of a size that keeps every branch of order one; rounded to ``store``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        rnd = lambda: torch.randn(shape, generator=g)                               # noqa: E731
        if "norm" in last:
            t = 1.0 + 0.2 * rnd()
        elif name.endswith("f.b"):
            t = -1.0 + 4.0 * torch.rand(shape, generator=g)          # gates between forgetting fast and slowly
        elif last == "lower":
            t = 0.9 * torch.rand(shape, generator=g)
        elif last == "b":
            t = 0.5 * rnd()
        elif last == "sink":
            t = rnd()
        elif name in ("embed", "side.embed"):
            t = rnd()
        elif last in ("q", "k", "uq", "uk") and "mix" in name:
            t = 2.0 * rnd() / math.sqrt(shape[-1])                   # scores of some size, so that the masks matter
        else:
            t = rnd() / math.sqrt(shape[-1])
        out[name] = t.to(store)
    return out
