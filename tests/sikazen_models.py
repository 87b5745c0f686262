"""Small Sikazen configurations for the tests, and a helper that writes their model folders from the plain
implementation's random weights.

S1: the three mixers in a row, the whole model run twice (a loop over all layers): six query heads over two, a window
    of 20 with blocks of 6 (blocks straddle pages of 4 and 16), half of a head rotated with scaled frequencies; latent
    attention of four heads; a recurrent layer of 3 heads of 16 x 32; a side table.
S2: sizes that no fast kernel takes (width 100, odd vocabulary, heads of 20 with values of 12, a latent of 24 + 6);
    a window of 7 that is shorter than its blocks of 9; as many key/value heads as heads; a layer without a
    feed-forward; no loop, no side table; a window without blocks; no rotation in one layer.
S3: a loop over the two middle layers, three times; twenty heads over one key/value head; a window of 1; blocks of
    one position; a recurrent layer whose value heads fill a state slice in part (vdim 24); an embedding scale that
    is no power of two.
S4: recurrent layers only (no pages at all), looped twice, with a side table.
S5: attention layers only (no state slot at all): no mask at all (every earlier key), a window of 33 with blocks of
    16 (a page's size), latent attention with one head.
"""
import json
import os

import plain_sikazen as PS


def _rot(base, dims, factor=None):
    r = {"base": base, "dims": dims}
    if factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def _attn(heads, kv_heads, dim, vdim, scale, rot=None, size=None, pool=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        m["rot"] = rot
    if size is not None:
        m["mask"] = {"size": size}
        if pool is not None:
            m["mask"]["pool"] = pool
    return m


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "scale": scale, "rot": _rot(base, rot_dim)}


def _hgrn2(heads, dim, vdim):
    return {"heads": heads, "dim": dim, "vdim": vdim}


def _layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


S1 = {"architecture": "Sikazen", "vocab": 200, "width": 64, "embedding": {"scale": 0.25}, "norm": {"eps": 1e-5},
      "token_side": {"dim": 8}, "loop": {"start": 0, "stop": 3, "times": 2},
      "layers": [_layer("attention", _attn(6, 2, 16, 32, 0.3, _rot(10000.0, 8, 2.0), 20, 6), 96),
                 _layer("latent_attention", _latent(4, 16, 16, 16, 32, 24, 0.2, 50000.0), 80),
                 _layer("hgrn2", _hgrn2(3, 16, 32), 96)]}
S2 = {"architecture": "Sikazen", "vocab": 333, "width": 100, "norm": {"eps": 1e-6},
      "layers": [_layer("attention", _attn(5, 5, 20, 12, 0.25, _rot(1000.0, 20), 7, 9), 60),
                 _layer("latent_attention", _latent(3, 10, 6, 14, 24, 9, 0.35, 100.0)),
                 _layer("attention", _attn(4, 2, 12, 20, 0.4, None, 11), 50),
                 _layer("hgrn2", _hgrn2(2, 10, 12), 40)]}
S3 = {"architecture": "Sikazen", "vocab": 256, "width": 128, "embedding": {"scale": 0.3}, "norm": {"eps": 3e-6},
      "token_side": {"dim": 5}, "loop": {"start": 1, "stop": 3, "times": 3},
      "layers": [_layer("attention", _attn(20, 1, 32, 16, 0.2, _rot(500.0, 32, 8.0), 1, 1), 72),
                 _layer("hgrn2", _hgrn2(4, 32, 24), 72),
                 _layer("attention", _attn(4, 4, 16, 16, 0.25, _rot(20000.0, 4), 48, 16), 64),
                 _layer("latent_attention", _latent(2, 32, 32, 32, 64, 48, 0.125, 10000.0), 72)]}
S4 = {"architecture": "Sikazen", "vocab": 150, "width": 80, "norm": {"eps": 1e-6}, "token_side": {"dim": 16},
      "loop": {"start": 0, "stop": 2, "times": 2},
      "layers": [_layer("hgrn2", _hgrn2(5, 16, 16), 64), _layer("hgrn2", _hgrn2(2, 40, 48), 48)]}
S5 = {"architecture": "Sikazen", "vocab": 1100, "width": 48, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
      "layers": [_layer("attention", _attn(3, 3, 48, 16, 0.15, _rot(10000.0, 48)), 64),
                 _layer("attention", _attn(4, 2, 16, 16, 0.25, _rot(10000.0, 16, 3.0), 33, 16)),
                 _layer("latent_attention", _latent(1, 48, 16, 64, 80, 32, 0.1, 300000.0), 32)]}
RAW = {"S1": S1, "S2": S2, "S3": S3, "S4": S4, "S5": S5}
SEED = {"S1": 5, "S2": 6, "S3": 7, "S4": 15, "S5": 9}


def write_model(name_or_cfg, out_dir: str, seed=None, weights=None):
    """Writes config.json and model.safetensors (bfloat16 values); returns (configuration dict, weights dict) as
    the plain implementation reads them."""
    import torch
    from infernum_amd.weights.safetensors_io import write_safetensors
    cfg = RAW[name_or_cfg] if isinstance(name_or_cfg, str) else name_or_cfg
    seed = (SEED[name_or_cfg] if isinstance(name_or_cfg, str) else 0) if seed is None else seed
    w = weights if weights is not None else PS.random_weights(cfg, seed)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      ((n, t.to(torch.bfloat16).contiguous()) for n, t in sorted(w.items())))
    return cfg, w
