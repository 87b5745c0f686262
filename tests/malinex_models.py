"""Small Malinex configurations for the tests, and a helper that writes their model folders from the plain
implementation's random weights.

X1: a recurrent layer with a dense feed-forward, an attention layer (four heads over two, a factor on the queries that
    steps every 16 positions) with six experts of which two are chosen and a shared expert of another width; then
    each of the two once more with the first run's tensors (``weights_of``): both kinds run twice with one set of
    tensors and two caches or states.
X2: sizes that no fast kernel takes (width 100, odd vocabulary, heads of 26 and 10, value heads of 24: a state slice
    filled in part); no ``kv_heads`` (as many as heads), no factor on the queries, no feed-forward in one layer; all
    five experts chosen, no shared expert; tau 1 (fast forgetting) and 30; no ``logit_scale``.
X3: twenty heads over one key/value head, keys of 32 and values of 64; the queries' factor steps at every position;
    seventy experts (more than a wave's lanes) of which one is chosen, a wide shared expert; a recurrent layer of four
    heads of 64 x 64, run twice.
X4: recurrent layers only (no pages at all), dense and then routed (a router in the last layer moves its own place only).
X5: attention layers only (no state slot at all), keys wider than values, one layer without a feed-forward.
"""
import json
import os

import plain_malinex as PM


def _gla(heads, dim, vdim, tau, rank):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def _attn(heads, kv_heads, dim, vdim, scale, q_temp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def _layer(kind, mixer, mlp=None, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


_x1_gla, _x1_att = _gla(2, 16, 32, 8.0, 8), _attn(4, 2, 16, 32, 0.25, (0.5, 16))
X1 = {"architecture": "Malinex", "vocab": 200, "width": 64, "max_positions": 256, "norm": {"eps": 1e-5},
      "logit_scale": 0.5,
      "layers": [_layer("gla", _x1_gla, _dense(96)), _layer("attention", _x1_att, _moe(6, 2, 40, 24)),
                 _layer("gla", _x1_gla, _dense(96), weights_of=0), _layer("attention", _x1_att, _moe(6, 2, 40, 24), weights_of=1)]}
X2 = {"architecture": "Malinex", "vocab": 333, "width": 100, "max_positions": 300, "norm": {"eps": 1e-6},
      "layers": [_layer("attention", _attn(5, None, 26, 10, 0.3)),
                 _layer("gla", _gla(3, 10, 24, 1.0, 3), _moe(5, 5, 30)),
                 _layer("gla", _gla(1, 40, 16, 30.0, 5), _dense(50))]}
_x3_gla = _gla(4, 64, 64, 4.0, 16)
X3 = {"architecture": "Malinex", "vocab": 256, "width": 128, "max_positions": 512, "norm": {"eps": 3e-6},
      "logit_scale": 2.0,
      "layers": [_layer("attention", _attn(20, 1, 32, 64, 0.2, (0.1, 1)), _moe(70, 1, 16, 64)),
                 _layer("gla", _x3_gla, _dense(72)), _layer("gla", _x3_gla, _dense(72), weights_of=1)]}
X4 = {"architecture": "Malinex", "vocab": 150, "width": 80, "max_positions": 400, "norm": {"eps": 1e-6},
      "logit_scale": 0.125,
      "layers": [_layer("gla", _gla(5, 16, 16, 2.0, 7), _dense(64)), _layer("gla", _gla(2, 32, 48, 16.0, 4), _moe(4, 3, 24, 24))]}
X5 = {"architecture": "Malinex", "vocab": 1100, "width": 48, "max_positions": 320, "norm": {"eps": 1e-5},
      "logit_scale": 1.5,
      "layers": [_layer("attention", _attn(3, 3, 48, 16, 0.15, (1.0, 100)), _dense(64)),
                 _layer("attention", _attn(4, 2, 16, 16, 0.25)),
                 _layer("attention", _attn(2, 1, 64, 32, 0.125, (0.25, 7)), _moe(3, 2, 32))]}
RAW = {"X1": X1, "X2": X2, "X3": X3, "X4": X4, "X5": X5}
SEED = {"X1": 5, "X2": 6, "X3": 7, "X4": 15, "X5": 9}


def write_model(name_or_cfg, out_dir: str, seed=None, weights=None, with_rank: bool = True):
    """Writes config.json and model.safetensors (bfloat16 values); returns (configuration dict, weights dict) as
    the plain implementation reads them.  ``with_rank`` False: the file's configuration does not tell the width of
    the decay logits' middle, as a file from elsewhere would not."""
    import copy
    import torch
    from infernum_amd.weights.safetensors_io import write_safetensors
    cfg = RAW[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    seed = (SEED[name_or_cfg] if isinstance(name_or_cfg, str) else 0) if seed is None else seed
    w = weights if weights is not None else PM.random_weights(cfg, seed)
    os.makedirs(out_dir, exist_ok=True)
    stored = copy.deepcopy(cfg)
    if not with_rank:
        for entry in stored["layers"]:
            entry["mixer"].pop("rank", None)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(stored, f)
    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      ((n, t.to(torch.bfloat16).contiguous()) for n, t in sorted(w.items())))
    return cfg, w
