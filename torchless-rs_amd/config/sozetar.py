"""`SozetarConfig`: the config.json of a Sozetar model, typed.

The file names its design in `architecture` (one string), the sizes `vocab` and
`width`, `norm.eps`, and `layers`, a list with one entry per layer: `type` (which
mixer), `mixer` (its sizes and constants) and `mlp` (the feed-forward, or null for a
layer without one).  Nothing about a layer is implied by another: every entry is
read on its own, so layers may differ in every size.

Mixer `attention`: `heads`, `kv_heads` (default: heads), `dim` (query and key size
per head), `vdim` (value size, default: dim), `scale` (the factor on q.k),
`mask.size` (the sliding window; no `mask`: every earlier position is seen),
`q_temp` = {`coef`, `every`} (the factor on q that grows with the position; absent:
none) and `kv_from` (the index of an earlier layer whose keys and values this layer
reads instead of making its own).  Feed-forward: `kind` (`dense`) and `ff`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, ModelConfig, take_float, take_int, take_obj as _obj

MAX_HEAD_DIM = 256          # the largest head the attention kernels take
NAME = "Sozetar"


@dataclass
class SozetarAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None
    q_temp_coef: Optional[float] = None
    q_temp_every: Optional[float] = None
    kv_from: Optional[int] = None

    @classmethod
    def from_dict(cls, m: Dict[str, Any], where: str, index: int) -> "SozetarAttention":
        def sized(key, **kw):
            try:
                return take_int(m, key, **kw)
            except ConfigError as e:
                raise ConfigError(f"{e} (in {where})") from None
        heads = sized("heads", required=True, minimum=1)
        kv_heads = sized("kv_heads", default=heads, minimum=1)
        dim = sized("dim", required=True, minimum=1)
        vdim = sized("vdim", default=dim, minimum=1)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if max(dim, vdim) > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: {where}: head sizes {dim}/{vdim} are not served (up to {MAX_HEAD_DIM})")
        mask = _obj(m, "mask", where)
        window = take_int(mask, "size", required=True, minimum=1) if mask is not None else None
        temp = _obj(m, "q_temp", where)
        coef = every = None
        if temp is not None:
            coef = take_float(temp, "coef", required=True)
            every = take_float(temp, "every", required=True, positive=True)
        kv_from = sized("kv_from", default=None, allow_none=True, minimum=0)
        if kv_from is not None and kv_from >= index:
            raise ConfigError(f"config.json: {where}: kv_from {kv_from} is not an earlier layer")
        return cls(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                   scale=take_float(m, "scale", required=True), window=window, q_temp_coef=coef,
                   q_temp_every=every, kv_from=kv_from)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.q_temp_coef is not None:
            every = self.q_temp_every
            d["q_temp"] = {"coef": self.q_temp_coef, "every": int(every) if every == int(every) else every}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass
class SozetarLayer:
    type: str
    mixer: SozetarAttention
    ff: Optional[int] = None          # None: no feed-forward
    mlp_kind: str = "dense"

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": self.mlp_kind, "ff": self.ff}}


MIXERS = {"attention": SozetarAttention}
MLP_KINDS = ("dense",)


@dataclass
class SozetarConfig(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    layers: List[SozetarLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    max_position_embeddings: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "SozetarConfig":
        norm = _obj(d, "norm", "the model", required=True)
        entries = d.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[SozetarLayer] = []
        for i, e in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}: no mixer of type {kind!r}; there are {sorted(MIXERS)}")
            mixer = MIXERS[kind].from_dict(_obj(e, "mixer", where, required=True), where, i)
            mlp = _obj(e, "mlp", where)
            ff, mlp_kind = None, "dense"
            if mlp is not None:
                mlp_kind = mlp.get("kind", "dense")
                if mlp_kind not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}: no feed-forward of kind {mlp_kind!r}; there are {MLP_KINDS}")
                ff = take_int(mlp, "ff", required=True, minimum=1)
            layers.append(SozetarLayer(type=kind, mixer=mixer, ff=ff, mlp_kind=mlp_kind))
        for i, l in enumerate(layers):
            src = l.mixer.kv_from
            if src is None:
                continue
            o = layers[src].mixer
            if o.kv_from is not None:
                raise ConfigError(f"config.json: layer {i} reads the keys of layer {src}, which has none of its own")
            if (o.kv_heads, o.dim, o.vdim) != (l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim):
                raise ConfigError(f"config.json: layer {i} reads the keys of layer {src}, whose head counts "
                                  "and sizes differ from its own")
        known = {"architecture", "architectures", "vocab", "width", "norm", "layers", "eos_token_id",
                 "max_position_embeddings", "torch_dtype"}
        eos = d.get("eos_token_id")
        eos_ids = [eos] if isinstance(eos, int) and not isinstance(eos, bool) else list(eos or [])
        return cls(architecture=NAME, extra={k: v for k, v in d.items() if k not in known},
                   vocab_size=take_int(d, "vocab", required=True, minimum=1),
                   hidden_size=take_int(d, "width", required=True, minimum=1),
                   norm_eps=take_float(norm, "eps", required=True, positive=True), layers=layers,
                   eos_token_ids=eos_ids,
                   max_position_embeddings=take_int(d, "max_position_embeddings", default=None, allow_none=True,
                                                    minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": NAME, "vocab": self.vocab_size, "width": self.hidden_size,
                             "norm": {"eps": self.norm_eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        d.update(self.extra)
        return d
