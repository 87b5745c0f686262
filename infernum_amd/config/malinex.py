"""Configuration of the Malinex decoder, read from its own config.json keys.

The file names its design in ``architecture`` and describes every layer by itself:
  vocab, width, max_positions (rows of the learned position table), norm.eps, logit_scale,
  layers[i].type        the mixer: "gla" | "attention",
  layers[i].mixer       gla: {heads, dim, vdim, tau} (and optionally rank, the width of the decay logits' middle, which a
                        file's tensors tell otherwise; random weights need it);
                        attention: {heads, kv_heads, dim, vdim, scale, q_temp: {coef, every}},
  layers[i].mlp         null | {kind: "dense", ff} | {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff}},
  layers[i].weights_of  j: the layer has no tensors of its own and runs with layer j's (mixer, feed-forward, norms,
                        gates), with a cache or state of its own.
Layers may differ in every size.  What a file does not mention is not there: no ``q_temp``, queries as the norm leaves
them; no ``shared``, the routed experts alone; no ``kv_heads``, as many as heads; no ``logit_scale``, 1.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .base import ConfigError, KeyReader

MALINEX_MODEL_TYPE = "Malinex"
MIXER_TYPES = ("gla", "attention")
MLP_KINDS = ("dense", "moe")


def _need(r: Optional[KeyReader], where: str, key: str) -> KeyReader:
    if r is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return r


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int                    # key (and query) channels a head
    vdim: int                   # values a head
    tau: float                  # alpha = sigmoid(z)^(1/tau)
    rank: Optional[int] = None  # width of the decay logits' middle; a file's tensors tell it when the key is absent

    @staticmethod
    def from_reader(r: KeyReader) -> "GlaConfig":
        return GlaConfig(heads=r.integer("heads", minimum=1), dim=r.integer("dim", minimum=1),
                         vdim=r.integer("vdim", minimum=1), tau=r.number("tau", positive=True),
                         rank=r.integer("rank", None, minimum=1))

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.rank is not None:
            out["rank"] = self.rank
        return out


@dataclass(frozen=True)
class SigmoidAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: Optional[float]        # None: no factor on the queries
    q_temp_every: int

    @staticmethod
    def from_reader(r: KeyReader) -> "SigmoidAttentionConfig":
        qt = r.obj("q_temp")
        heads = r.integer("heads", minimum=1)
        m = SigmoidAttentionConfig(
            heads=heads, kv_heads=r.integer("kv_heads", heads, minimum=1), dim=r.integer("dim", minimum=1),
            vdim=r.integer("vdim", minimum=1), scale=r.number("scale", positive=True),
            q_temp_coef=qt.number("coef") if qt is not None else None,
            q_temp_every=qt.integer("every", minimum=1) if qt is not None else 0)
        if m.heads % m.kv_heads:
            raise ConfigError(f"{r.where}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        return m

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.q_temp_coef is not None:
            out["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return out


@dataclass(frozen=True)
class MalinexMlpConfig:
    kind: str
    ff: int                             # dense: the middle's width; moe: an expert's
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None     # the expert that every token takes; None: there is none

    @staticmethod
    def from_reader(r: KeyReader) -> "MalinexMlpConfig":
        kind = r.string("kind", choices=MLP_KINDS)
        if kind == "dense":
            return MalinexMlpConfig(kind, r.integer("ff", minimum=1))
        router, expert, shared = _need(r.obj("router"), r.where, "router"), _need(r.obj("expert"), r.where, "expert"), r.obj("shared")
        m = MalinexMlpConfig(kind, expert.integer("ff", minimum=1), router.integer("experts", minimum=1),
                             router.integer("top", minimum=1),
                             shared.integer("ff", minimum=1) if shared is not None else None)
        if m.top > m.experts:
            raise ConfigError(f"{r.where}: a token cannot take {m.top} of {m.experts} experts")
        return m

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        out = {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class MalinexLayerConfig:
    type: str
    mixer: Union[GlaConfig, SigmoidAttentionConfig]
    mlp: Optional[MalinexMlpConfig]
    weights_of: Optional[int] = None

    def to_dict(self) -> dict:
        out = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


@dataclass(frozen=True)
class MalinexConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    layers: Tuple[MalinexLayerConfig, ...]
    logit_scale: float = 1.0
    model_type: str = MALINEX_MODEL_TYPE

    # what the generation entry points ask of every configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    bos_token_id = None
    eos_token_id = None

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs with."""
        w = self.layers[i].weights_of
        return i if w is None else w

    @staticmethod
    def from_dict(raw: Mapping[str, Any], where: str = "config.json") -> "MalinexConfig":
        r = KeyReader(raw, where)
        norm = _need(r.obj("norm"), where, "norm")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            lr = KeyReader(entry, f"{where}:layers[{i}]")
            kind = lr.string("type", choices=MIXER_TYPES)
            mr = _need(lr.obj("mixer"), lr.where, "mixer")
            mixer = GlaConfig.from_reader(mr) if kind == "gla" else SigmoidAttentionConfig.from_reader(mr)
            mlp = lr.obj("mlp")
            layers.append(MalinexLayerConfig(kind, mixer, MalinexMlpConfig.from_reader(mlp) if mlp is not None else None,
                                             lr.integer("weights_of", None, minimum=0)))
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is None:
                continue
            if j >= len(layers) or j == i or layers[j].weights_of is not None:
                raise ConfigError(f"{where}:layers[{i}]: weights_of {j} does not name a layer with tensors of its own")
            if (layers[j].type, layers[j].mixer, layers[j].mlp) != (layer.type, layer.mixer, layer.mlp):
                raise ConfigError(f"{where}:layers[{i}]: a layer that runs with layer {j}'s tensors must have its sizes")
        return MalinexConfig(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            max_positions=r.integer("max_positions", minimum=1), norm_eps=norm.number("eps", positive=True),
            layers=tuple(layers), logit_scale=r.number("logit_scale", 1.0))

    def to_dict(self) -> dict:
        return {"architecture": self.model_type, "vocab": self.vocab, "width": self.width,
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale,
                "layers": [l.to_dict() for l in self.layers]}
