"""The Malinex decoder as a ModelSpec: layers with a norm before and after each sublayer and a sigmoid gate on each
sublayer's result (``sandwich``); the mixer is gated linear attention (``gla``) or attention with sigmoid weights
(``sigmoid_attention``); the feed-forward is dense (erf GELU), routed experts without a gate (squared relu, a
softmax over all experts, a correction that moves the choice only, a shared expert) or absent; a learned vector per
position is added to the embedding; a layer may run with another layer's tensors and a cache or state of its own;
the logits are multiplied by a constant.  Tensor names: ``embed``, ``pos``, ``final.norm``, ``head``,
``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.rg1|rg2`` (+ ``.b``), ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.malinex import MALINEX_MODEL_TYPE, MalinexConfig
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

EXPERT_ACTIVATION = "relu_squared"      # fixed by the design, like the dense feed-forward's erf GELU
DENSE_ACTIVATION = "gelu"


def malinex_model_spec(cfg: MalinexConfig, init_std: float = 0.05) -> ModelSpec:
    W = cfg.width

    def norm(prefix: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": W, "eps": cfg.norm_eps, "init": ("uniform", 0.8, 1.2), "name": ""}, prefix)

    def gate(prefix: str) -> tuple:
        return ("branch_gate", PartSpec("sigmoid_linear", {"hidden_size": W, "name": "", "bias_name": ".b",
                                                           "init_std": init_std}, prefix))

    layers, spec_index = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        spec_index[i] = len(layers)
        p, m = f"l{i}.", layer.mixer
        if layer.type == "attention":
            q_temp = {"coef": m.q_temp_coef, "every": m.q_temp_every} if m.q_temp_coef is not None else None
            mixer = PartSpec("sigmoid_attention", {
                "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "norm_eps": cfg.norm_eps, "q_temp": q_temp,
                "init_std": init_std}, p + "mix.")
        else:
            mixer = PartSpec("gla", {"hidden_size": W, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                                     "tau": m.tau, "decay_rank": m.rank, "norm_eps": cfg.norm_eps,
                                     "init_std": init_std}, p + "mix.")
        ff, mlp = None, layer.mlp
        if mlp is not None and mlp.kind == "dense":
            ff = PartSpec("dense", {"hidden_size": W, "intermediate_size": mlp.ff, "activation": DENSE_ACTIVATION,
                                    "names": ("up", "down"), "init_std": init_std}, p + "mlp.")
        elif mlp is not None:
            ff = PartSpec("routed_experts", {
                "hidden_size": W, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top,
                "gated": False, "activation": EXPERT_ACTIVATION, "router": "softmax_top", "shared_ff": mlp.shared_ff,
                "init_std": init_std}, p + "mlp.")
        extra = {"mixer_post_norm": norm(p + "norm1b"), "mixer_gate": gate(p + "rg1")}
        if ff is not None:
            extra.update({"feed_forward_post_norm": norm(p + "norm2b"), "feed_forward_gate": gate(p + "rg2")})
        layers.append(LayerSpec(block="sandwich", mixer=mixer, feed_forward=ff, mixer_norm=norm(p + "norm1"),
                                feed_forward_norm=norm(p + "norm2") if ff is not None else None, extra=extra))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=W,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed", "init_std": 1.0,
                                     "position_table": {"name": "pos", "rows": cfg.max_positions, "init_std": 0.5}}, ""),
        layers=layers,
        # a layer that runs with another's tensors is a second run of that layer, with a cache and state of its own
        schedule=[ScheduleEntry(spec_index[cfg.owner(i)]) for i in range(len(cfg.layers))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "", "scale": cfg.logit_scale,
                                 "init_std": W ** -0.5}, "head"),
        max_position=cfg.max_positions,
    )


register_architecture(MALINEX_MODEL_TYPE, MalinexConfig, malinex_model_spec)
