"""Configuration of the Sikazen decoder, read from its own config.json keys.

The file names its design in ``architecture`` and describes every layer by itself:
  vocab, width, embedding.scale, norm.eps,
  token_side       null | {dim}: every layer reads ``dim`` values of a second table's row of the token,
  loop             null | {start, stop, times}: layers start .. stop-1 run ``times`` times in a row,
  layers[i].type   the mixer: "attention" | "latent_attention" | "hgrn2",
  layers[i].mixer  attention: {heads, kv_heads, dim, vdim, scale, rot: {base, dims, scaling: {factor}},
                   mask: {size, pool}};
                   latent_attention: {heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot: {base, dims}};
                   hgrn2: {heads, dim, vdim},
  layers[i].mlp    null | {kind: "dense", ff}.
Layers may differ in every size.  What a file does not mention is not there: no ``loop``, no repetition; no
``token_side``, no second table; no ``mask``, all earlier keys one by one; no ``rot``, no rotation; no
``rot.scaling``, the plain frequencies.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from .base import ConfigError, KeyReader

SIKAZEN_MODEL_TYPE = "Sikazen"
MIXER_TYPES = ("attention", "latent_attention", "hgrn2")
MLP_KINDS = ("dense",)


def _need(r: Optional[KeyReader], where: str, key: str) -> KeyReader:
    if r is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return r


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    factor: float = 1.0         # every frequency is divided by it

    @staticmethod
    def from_reader(r: Optional[KeyReader], most: int) -> Optional["Rotation"]:
        if r is None:
            return None
        sc = r.obj("scaling")
        rot = Rotation(r.number("base", positive=True), r.integer("dims", minimum=0),
                       sc.number("factor", positive=True) if sc is not None else 1.0)
        if rot.dims > most or rot.dims % 2:
            raise ConfigError(f"{r.where}: dims must be even and at most {most}, got {rot.dims}")
        return rot if rot.dims > 0 else None

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            out["scaling"] = {"factor": self.factor}
        return out


@dataclass(frozen=True)
class PooledAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation]
    window: Optional[int]       # single keys a query sees, itself included; None: all earlier keys
    pool: Optional[int]         # keys of a block that is seen through its mean once it lies before the window

    @staticmethod
    def from_reader(r: KeyReader) -> "PooledAttentionConfig":
        mask = r.obj("mask")
        m = PooledAttentionConfig(
            heads=r.integer("heads", minimum=1), kv_heads=r.integer("kv_heads", minimum=1),
            dim=r.integer("dim", minimum=1), vdim=r.integer("vdim", minimum=1), scale=r.number("scale", positive=True),
            rot=Rotation.from_reader(r.obj("rot"), r.integer("dim", minimum=1)),
            window=mask.integer("size", None, minimum=1) if mask is not None else None,
            pool=mask.integer("pool", None, minimum=1) if mask is not None else None)
        if m.heads % m.kv_heads:
            raise ConfigError(f"{r.where}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        if m.pool is not None and m.window is None:
            raise ConfigError(f"{r.where}: mask.pool needs mask.size")
        return m

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.window is not None:
            out["mask"] = {"size": self.window}
            if self.pool is not None:
                out["mask"]["pool"] = self.pool
        return out


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                    # values of a head's query and key that are not rotated
    rot_dim: int                # rotated values, shared by the heads on the key side
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Optional[Rotation]

    @staticmethod
    def from_reader(r: KeyReader) -> "LatentAttentionConfig":
        rot_dim = r.integer("rot_dim", minimum=0)
        m = LatentAttentionConfig(
            heads=r.integer("heads", minimum=1), dim=r.integer("dim", minimum=1), rot_dim=rot_dim,
            vdim=r.integer("vdim", minimum=1), kv_rank=r.integer("kv_rank", minimum=1),
            q_rank=r.integer("q_rank", minimum=1), scale=r.number("scale", positive=True),
            rot=Rotation.from_reader(r.obj("rot"), rot_dim))
        return m

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
               "kv_rank": self.kv_rank, "q_rank": self.q_rank, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class Hgrn2Config:
    heads: int
    dim: int
    vdim: int

    @staticmethod
    def from_reader(r: KeyReader) -> "Hgrn2Config":
        return Hgrn2Config(r.integer("heads", minimum=1), r.integer("dim", minimum=1), r.integer("vdim", minimum=1))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}


_MIXERS = {"attention": PooledAttentionConfig, "latent_attention": LatentAttentionConfig, "hgrn2": Hgrn2Config}


@dataclass(frozen=True)
class MlpConfig:
    kind: str
    ff: int

    def to_dict(self) -> dict:
        return {"kind": self.kind, "ff": self.ff}


@dataclass(frozen=True)
class SikazenLayerConfig:
    type: str
    mixer: Union[PooledAttentionConfig, LatentAttentionConfig, Hgrn2Config]
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class SikazenConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[SikazenLayerConfig, ...]
    loop: Optional[LoopConfig] = None
    side_dim: Optional[int] = None
    model_type: str = SIKAZEN_MODEL_TYPE

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

    bos_token_id = None
    eos_token_id = None

    def layer_runs(self) -> Tuple[Tuple[int, int], ...]:
        """(layer, pass of the loop that the run belongs to: 0 outside the loop and in its first pass) in the order
        the layers run."""
        n = len(self.layers)
        if self.loop is None or self.loop.times <= 1 or self.loop.stop <= self.loop.start:
            return tuple((i, 0) for i in range(n))
        a, b = self.loop.start, self.loop.stop
        runs = [(i, 0) for i in range(a)]
        for t in range(self.loop.times):
            runs += [(i, t) for i in range(a, b)]
        return tuple(runs + [(i, 0) for i in range(b, n)])

    @staticmethod
    def from_dict(raw: Mapping[str, Any], where: str = "config.json") -> "SikazenConfig":
        r = KeyReader(raw, where)
        emb, norm = r.obj("embedding"), _need(r.obj("norm"), where, "norm")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            lr = KeyReader(entry, f"{where}:layers[{i}]")
            kind = lr.string("type", choices=MIXER_TYPES)
            mixer = _MIXERS[kind].from_reader(_need(lr.obj("mixer"), lr.where, "mixer"))
            mlp = lr.obj("mlp")
            layers.append(SikazenLayerConfig(kind, mixer, MlpConfig(mlp.string("kind", choices=MLP_KINDS),
                                                                  mlp.integer("ff", minimum=1)) if mlp is not None else None))
        loop, lp = None, r.obj("loop")
        if lp is not None:
            loop = LoopConfig(lp.integer("start", minimum=0), lp.integer("stop", minimum=0), lp.integer("times", minimum=1))
            if not loop.start <= loop.stop <= len(layers):
                raise ConfigError(f"{where}: loop {loop.start} .. {loop.stop} does not lie within the {len(layers)} layers")
        side = r.obj("token_side")
        return SikazenConfig(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            embedding_scale=emb.number("scale", 1.0) if emb is not None else 1.0,
            norm_eps=norm.number("eps", positive=True), layers=tuple(layers), loop=loop,
            side_dim=side.integer("dim", minimum=1) if side is not None else None)

    def to_dict(self) -> dict:
        out = {"architecture": self.model_type, "vocab": self.vocab, "width": self.width,
               "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
               "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": l.mlp.to_dict() if l.mlp else None}
                          for l in self.layers]}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.side_dim is not None:
            out["token_side"] = {"dim": self.side_dim}
        return out
