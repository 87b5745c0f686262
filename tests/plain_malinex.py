"""The Malinex decoder, plainly: whole sequences, no cache, float64, one function per mechanism.

It shares nothing with the package: a model is a configuration (the dict that config.json holds) and a dict of
tensors by their names in a file.  ``round_to=torch.bfloat16`` rounds what a bfloat16 engine stores between its
kernels, which tells how far rounding alone moves the logits.

Notation.  W: the stream's width.  A layer takes the stream x [T, W]:

    a = N1(x);   x <- x + N1b( mixer(a) * sigmoid(R1 a + r1) )
    f = N2(x);   x <- x + N2b( ff(f)    * sigmoid(R2 f + r2) )          (when the layer has a feed-forward)

with N(y) = y / sqrt(mean(y^2) + eps) * w.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Mapping, Optional

import torch

F64 = torch.float64


def _r(x: torch.Tensor, round_to) -> torch.Tensor:
    return x if round_to is None else x.to(round_to).to(F64)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * sigmoid(x)


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    return torch.clamp(x, min=0.0) ** 2


def embed(tokens: torch.Tensor, table: torch.Tensor, positions: torch.Tensor, pos_table: torch.Tensor) -> torch.Tensor:
    """Row of the token plus the learned row of its position."""
    return table[tokens] + pos_table[positions]


# ------------------------------------------------------------------------------------------------ mixers
def gla_decays(a: torch.Tensor, wa1: torch.Tensor, wa2: torch.Tensor, ba2: torch.Tensor, tau: float,
               round_to=None) -> torch.Tensor:
    """log(alpha) per token and key channel [T, heads * dim]: alpha = sigmoid(z)^(1/tau), z through a narrow middle."""
    z = _r(a @ wa1.T, round_to) @ wa2.T + ba2
    return -torch.log1p(torch.exp(-z)) / tau


def gla_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_alpha: torch.Tensor,
                   state: Optional[torch.Tensor] = None):
    """One head, token after token.  q, k, log_alpha [T, dim], v [T, vdim]; the state S [dim, vdim] starts at zero.
    S <- diag(alpha_t) S + k_t v_t^T;  o_t = S^T q_t.  Returns (o [T, vdim], S)."""
    T, dim = q.shape
    S = torch.zeros((dim, v.shape[1]), dtype=F64) if state is None else state.clone()
    out = torch.empty((T, v.shape[1]), dtype=F64)
    for t in range(T):
        S = torch.exp(log_alpha[t])[:, None] * S + k[t][:, None] * v[t][None, :]
        out[t] = S.T @ q[t]
    return out, S


def gla_mixer(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float, round_to=None) -> torch.Tensor:
    heads, dim, vdim, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = a.shape[0]
    q = _r(a @ w[p + "q"].T, round_to) * dim ** -0.5
    k = _r(a @ w[p + "k"].T, round_to)
    v = _r(a @ w[p + "v"].T, round_to)
    gate = silu(_r(a @ w[p + "g"].T, round_to))
    la = gla_decays(a, w[p + "a1"], w[p + "a2"], w[p + "a2.b"], tau, round_to)
    o = torch.empty((T, heads, vdim), dtype=F64)
    for h in range(heads):
        sl = slice(h * dim, (h + 1) * dim)
        o[:, h], _ = gla_recurrence(q[:, sl], k[:, sl], v[:, h * vdim:(h + 1) * vdim], la[:, sl])
    o = rms_norm(o, w[p + "norm"], eps).reshape(T, heads * vdim)
    return _r(_r(o * gate, round_to) @ w[p + "o"].T, round_to)


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.div(positions + 1, every, rounding_mode="floor").to(F64) + 1.0)


def sigmoid_attention_weights(q: torch.Tensor, k: torch.Tensor, scale: float, r1: float, r2: float, pb: float,
                              offset: int = 0) -> torch.Tensor:
    """One head.  q [Tq, dim] at positions offset .. offset+Tq-1, k [Tk, dim] at 0 .. Tk-1.  The weight of key j for
    the query at i >= j is sigmoid(scale q_i.k_j - r1 ln(1 + r2 (i - j)) + pb); later keys weigh nothing; no
    normalisation over the keys."""
    Tq, Tk = q.shape[0], k.shape[0]
    i = torch.arange(offset, offset + Tq, dtype=F64)[:, None]
    j = torch.arange(Tk, dtype=F64)[None, :]
    dist = torch.clamp(i - j, min=0.0)
    s = (q @ k.T) * scale - r1 * torch.log1p(r2 * dist) + pb
    return torch.where(j <= i, sigmoid(s), torch.zeros((), dtype=F64))


def attention_mixer(a: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, m: Mapping, eps: float,
                    round_to=None) -> torch.Tensor:
    H, G, dim, vdim = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    T = a.shape[0]
    pos = torch.arange(T)
    q = _r(a @ w[p + "q"].T + w[p + "q.b"], round_to)
    k = _r(a @ w[p + "k"].T + w[p + "k.b"], round_to)
    v = _r(a @ w[p + "v"].T + w[p + "v.b"], round_to)
    q = rms_norm(q, w[p + "q.norm"], eps)               # over all heads' values at once
    k = rms_norm(k, w[p + "k.norm"], eps)
    qt = m.get("q_temp")
    if qt is not None:
        q = q * query_temperature(pos, float(qt["coef"]), int(qt["every"]))[:, None]
    q, k = _r(q, round_to), _r(k, round_to)
    gate = sigmoid(a @ w[p + "g"].T)                     # [T, H]
    out = torch.empty((T, H, vdim), dtype=F64)
    for h in range(H):
        g = h // (H // G)
        wts = sigmoid_attention_weights(q[:, h * dim:(h + 1) * dim], k[:, g * dim:(g + 1) * dim], float(m["scale"]),
                                        float(w[p + "r1"][h]), float(w[p + "r2"][h]), float(w[p + "pb"][h]))
        out[:, h] = (wts @ v[:, g * vdim:(g + 1) * vdim]) * gate[:, h:h + 1]
    return _r(_r(out.reshape(T, H * vdim), round_to) @ w[p + "o"].T, round_to)


# ------------------------------------------------------------------------------------------ feed-forwards
def small_ff(f: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act: Callable, round_to=None) -> torch.Tensor:
    return _r(act(_r(f @ up.T, round_to)), round_to) @ down.T


def router(f: torch.Tensor, wr: torch.Tensor, correction: torch.Tensor, top: int, margins: Optional[List] = None,
           at_stake: float = 0.01):
    """-> (chosen [T, top], weights [T, top]): softmax over all experts; the choice goes by score + correction, the
    weights are the chosen scores themselves over their sum.  ``margins`` collects, per token, by how much the last
    chosen expert beats the first that is not, as a fraction of its own choice score; a token whose last chosen
    expert weighs less than ``at_stake`` counts as sure (margin 1): the other choice would change next to nothing."""
    s = torch.softmax(f @ wr.T, dim=-1)
    chosen = torch.topk(s + correction, top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    weights = picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)
    if margins is not None and top < s.shape[1]:
        c = torch.sort(s + correction, dim=-1, descending=True).values
        gap = (c[:, top - 1] - c[:, top]) / c[:, top - 1].abs().clamp_min(1e-30)
        last = torch.gather(weights, 1, torch.argmin(torch.gather(s + correction, 1, chosen), dim=-1, keepdim=True))[:, 0]
        margins.append(torch.where(last < at_stake, torch.ones_like(gap), gap))
    return chosen, weights


def routed_ff(f: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mlp: Mapping, round_to=None,
              margins: Optional[List] = None) -> torch.Tensor:
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    chosen, weights = router(f, w[p + "router"], w[p + "correction"], top, margins)
    out = torch.zeros((f.shape[0], w[p + "e0.down"].shape[0]), dtype=F64)
    for t in range(f.shape[0]):
        for c in range(top):
            e = int(chosen[t, c])
            out[t] += weights[t, c] * small_ff(f[t:t + 1], w[p + f"e{e}.up"], w[p + f"e{e}.down"], relu_squared, round_to)[0]
    if mlp.get("shared") is not None:
        out = out + small_ff(f, w[p + "shared.up"], w[p + "shared.down"], relu_squared, round_to)
    return out


def feed_forward(f: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, mlp: Mapping, round_to=None,
                 margins: Optional[List] = None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return _r(small_ff(f, w[p + "up"], w[p + "down"], gelu_erf, round_to), round_to)
    return routed_ff(f, w, p, mlp, round_to, margins)


# --------------------------------------------------------------------------------------------- the model
def layer(x: torch.Tensor, w: Mapping[str, torch.Tensor], p: str, entry: Mapping, eps: float, round_to=None,
          margins: Optional[List] = None) -> torch.Tensor:
    a = _r(rms_norm(x, w[p + "norm1"], eps), round_to)
    mix = gla_mixer if entry["type"] == "gla" else attention_mixer
    y = mix(a, w, p + "mix.", entry["mixer"], eps, round_to) * sigmoid(a @ w[p + "rg1"].T + w[p + "rg1.b"])
    x = x + rms_norm(y, w[p + "norm1b"], eps)
    if entry.get("mlp") is not None:
        f = _r(rms_norm(x, w[p + "norm2"], eps), round_to)
        y = feed_forward(f, w, p + "mlp.", entry["mlp"], round_to, margins) * sigmoid(f @ w[p + "rg2"].T + w[p + "rg2.b"])
        x = x + rms_norm(y, w[p + "norm2b"], eps)
    return x


def forward(config: Mapping, weights: Mapping[str, torch.Tensor], tokens, round_to=None,
            streams: Optional[List[torch.Tensor]] = None, layers: Optional[int] = None,
            margins: Optional[List] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its first token.  ``streams`` collects the stream after every layer;
    ``layers`` stops after so many; ``margins`` collects the routers' margins (see ``router``)."""
    w = {k: v.to(F64) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(config["norm"]["eps"])
    x = embed(tokens, w["embed"], torch.arange(tokens.numel()), w["pos"])
    for i, entry in enumerate(config["layers"][:layers]):
        x = layer(x, w, f"l{entry.get('weights_of', i)}.", entry, eps, round_to, margins)
        if streams is not None:
            streams.append(x.clone())
    x = _r(rms_norm(x, w["final.norm"], eps), round_to)
    return (x @ w["head"].T) * float(config.get("logit_scale", 1.0))


# ------------------------------------------------------------------------------------------- test models
def tensor_shapes(cfg: Mapping) -> Dict[str, tuple]:
    """Name -> shape of every tensor a file of this configuration holds (a gla mixer's ``rank`` is the width of its
    decay logits' middle)."""
    W, out = cfg["width"], {}
    out["embed"], out["pos"] = (cfg["vocab"], W), (cfg["max_positions"], W)
    for i, entry in enumerate(cfg["layers"]):
        if "weights_of" in entry:
            continue
        p, m = f"l{i}.", entry["mixer"]
        for n in ("norm1", "norm1b"):
            out[p + n] = (W,)
        out[p + "rg1"], out[p + "rg1.b"] = (W, W), (W,)
        if entry["type"] == "gla":
            nq, nv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (nq, W), p + "mix.k": (nq, W), p + "mix.v": (nv, W), p + "mix.g": (nv, W),
                        p + "mix.o": (W, nv), p + "mix.norm": (m["vdim"],), p + "mix.a1": (m["rank"], W),
                        p + "mix.a2": (nq, m["rank"]), p + "mix.a2.b": (nq,)})
        else:
            H, G = m["heads"], m.get("kv_heads", m["heads"])
            nq, nk, nv = H * m["dim"], G * m["dim"], G * m["vdim"]
            out.update({p + "mix.q": (nq, W), p + "mix.q.b": (nq,), p + "mix.k": (nk, W), p + "mix.k.b": (nk,),
                        p + "mix.v": (nv, W), p + "mix.v.b": (nv,), p + "mix.q.norm": (nq,), p + "mix.k.norm": (nk,),
                        p + "mix.r1": (H,), p + "mix.r2": (H,), p + "mix.pb": (H,), p + "mix.g": (H, W),
                        p + "mix.o": (W, H * m["vdim"])})
        mlp = entry.get("mlp")
        if mlp is None:
            continue
        for n in ("norm2", "norm2b"):
            out[p + n] = (W,)
        out[p + "rg2"], out[p + "rg2.b"] = (W, W), (W,)
        if mlp["kind"] == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"] = (mlp["ff"], W), (W, mlp["ff"])
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(E):
                out[p + f"mlp.e{e}.up"], out[p + f"mlp.e{e}.down"] = (ff, W), (W, ff)
            out[p + "mlp.router"], out[p + "mlp.correction"] = (E, W), (E,)
            if mlp.get("shared") is not None:
                sf = mlp["shared"]["ff"]
                out[p + "mlp.shared.up"], out[p + "mlp.shared.down"] = (sf, W), (W, sf)
    out["final.norm"], out["head"] = (W,), (cfg["vocab"], W)
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
        elif name.endswith("a2.b"):
            t = 1.0 + 3.0 * torch.rand(shape, generator=g)           # decays between forgetting fast and slowly
        elif last == "b":
            t = 0.5 * rnd()
        elif last == "r1":
            t = 0.2 + 0.8 * torch.rand(shape, generator=g)
        elif last == "r2":
            t = 0.05 + 0.5 * torch.rand(shape, generator=g)
        elif last == "pb":
            t = -3.0 + 2.0 * torch.rand(shape, generator=g)
        elif last == "correction":
            t = 0.05 * rnd()
        elif name == "embed":
            t = rnd()
        elif name == "pos":
            t = 0.5 * rnd()
        elif last == "router":
            t = 6.0 * rnd() / math.sqrt(shape[-1])
        else:
            t = rnd() / math.sqrt(shape[-1])
        out[name] = t.to(store)
    return out
