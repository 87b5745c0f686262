"""The Sikazen decoder as a ModelSpec: layers whose mixer and feed-forward run side by side behind a norm each of
the same stream (``parallel``), every norm with a single number as its weight; the mixer is attention over a window
of keys and pooled blocks before it (``pooled_window_attention``), latent attention with a query latent and a sink per
head (``latent_attention``), or HGRN2 (``hgrn2``); a gated feed-forward or none; after the sublayers a layer adds an
input of the tokens themselves, read from its part of a second table (``gated_table``); a stretch of layers may run
several times with the same tensors, every pass with a cache and state of its own, the embedding's rows added to
the stream before every pass but the first.  Tensor names: ``embed``, ``side.embed``, ``final.norm``, ``head``,
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.gate|proj|norm``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.sikazen import SIKAZEN_MODEL_TYPE, SikazenConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _rope(rot, head_dim: int, pairing: str) -> dict:
    if rot is None:
        return {"kind": "none"}
    scaling = {"rope_type": "linear", "factor": rot.factor} if rot.factor != 1.0 else None
    return {"kind": "rope", "params": {"head_dim": head_dim, "theta": rot.base, "rotary_dim": rot.dims,
                                       "scaling": scaling, "pairing": pairing}}


def sikazen_model_spec(cfg: SikazenConfig, init_std: float = 0.05) -> ModelSpec:
    W = cfg.width

    def norm(prefix: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "init": ("uniform", 0.8, 1.2), "name": "",
                                    "scalar": True}, prefix)

    runs = cfg.layer_runs()
    loops = any(t > 0 for _, t in runs)
    side_cols = cfg.side_dim * len(cfg.layers) if cfg.side_dim else 0
    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        if layer.type == "attention":
            mixer = PartSpec("pooled_window_attention", {
                "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "position": _rope(m.rot, m.dim, "half"), "window": m.window,
                "pool": m.pool, "bias": True, "qk_unit_norm": True, "norm_eps": cfg.norm_eps, "init_std": init_std},
                p + "mix.")
        elif layer.type == "latent_attention":
            mixer = PartSpec("latent_attention", {
                "hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
                "rank": m.kv_rank, "q_rank": m.q_rank, "norm_eps": cfg.norm_eps, "scale": m.scale,
                "position": _rope(m.rot, m.rot_dim + m.kv_rank, "neighbours"), "window": None, "gate": False,
                "sink": True, "init_std": init_std}, p + "mix.")
        else:
            mixer = PartSpec("hgrn2", {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                                       "norm_eps": cfg.norm_eps, "init_std": init_std}, p + "mix.")
        ff = None
        if layer.mlp is not None:
            ff = PartSpec("swiglu", {"hidden_size": W, "intermediate_size": layer.mlp.ff, "init_std": init_std,
                                     "names": ("gate", "up", "down")}, p + "mlp.")
        extra = {}
        if loops and i == cfg.loop.start:           # every pass but the first enters through this layer
            extra["stream_in"] = ("stream_in", PartSpec("add_embedding", {"hidden_size": W}, ""))
        if cfg.side_dim:
            extra["token_input"] = ("token_input", PartSpec("gated_table", {
                "hidden_size": W, "vocab_size": cfg.vocab, "dim": cfg.side_dim, "column": i * cfg.side_dim,
                "columns": side_cols, "eps": cfg.norm_eps, "table": "side.embed",
                "names": ("embed", "gate", "proj", "norm"), "init_std": init_std}, p + "side."))
        layers.append(LayerSpec(block="parallel", mixer=mixer, feed_forward=ff, mixer_norm=norm(p + "norm1"),
                                feed_forward_norm=norm(p + "norm2") if ff is not None else None, extra=extra))
    embedding = {"vocab_size": cfg.vocab, "hidden_size": W, "scale": cfg.embedding_scale, "name": "embed",
                 "init_std": 1.0 / max(cfg.embedding_scale, 1e-3), "keep_output": "fp32" if loops else False}
    if cfg.side_dim:
        embedding["extra_tables"] = {"side.embed": {"cols": side_cols, "init_std": 1.0}}
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=W, embedding=PartSpec("token", embedding, ""),
        layers=layers, schedule=[ScheduleEntry(i, pass_index=t) for i, t in runs],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "", "init_std": W ** -0.5}, "head"),
        # a layer without a feed-forward has no use for a second norm, whether the file holds one or not
        ignored_tensors=tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.mlp is None),
    )


register_architecture(SIKAZEN_MODEL_TYPE, SikazenConfig, sikazen_model_spec)
