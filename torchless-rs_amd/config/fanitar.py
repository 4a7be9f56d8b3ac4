"""`FanitarConfig`: the config.json of a Fanitar model, typed.

The file names its design in `architecture`, the sizes `vocab` and `width`, `norm.eps`,
`embedding.scale` (the factor on an embedding row), `logit_scale` (the factor on the
logits), `layers`, a list with one entry per layer, and `loop` = {`start`, `stop`, `times`}:
layers start .. stop - 1 are gone through `times` times in a row with the same weights
(absent: every layer runs once).  A layer's entry has `type` (which mixer), `mixer` (its
sizes and constants) and `mlp` (the feed-forward, or null for a layer without one); every
entry is read on its own, so layers may differ in every size.

Mixer `latent_attention`: `heads`, `dim` (query and key size per head), `vdim` (value size,
default: dim), `q_rank` and `kv_rank` (the sizes of the two latents), `scale` (the factor on
q.k) and `mask.size` (the sliding window; no `mask`: every earlier position is seen).
Mixer `attention` (differential, two maps a head): `heads`, `kv_heads` (default: heads), `dim`
(the size of ONE map's query and key), `vdim` (default: dim), `scale`, `diff` (the constant
in lambda, whose complement scales the head's output), `rot` = {`base`, `dims`} (the rotated
channels of each map; absent: no rotation) and `mask.size`.
Feed-forward: `kind` (`dense`), `ff` and `limit` (the clamp of gate and up).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, ModelConfig, take_float, take_int, take_obj

MAX_HEAD_DIM = 256          # the largest head the attention kernels take
NAME = "Fanitar"


def _sized(m, key, where, **kw):
    try:
        return take_int(m, key, **kw)
    except ConfigError as e:
        raise ConfigError(f"{e} (in {where})") from None


def _window(m, where) -> Optional[int]:
    mask = take_obj(m, "mask", where)
    return take_int(mask, "size", required=True, minimum=1) if mask is not None else None


@dataclass
class FanitarLatentAttention:
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: Optional[int] = None

    @classmethod
    def from_dict(cls, m: Dict[str, Any], where: str) -> "FanitarLatentAttention":
        heads = _sized(m, "heads", where, required=True, minimum=1)
        dim = _sized(m, "dim", where, required=True, minimum=1)
        vdim = _sized(m, "vdim", where, default=dim, minimum=1)
        if max(dim, vdim) > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: {where}: head sizes {dim}/{vdim} are not served (up to {MAX_HEAD_DIM})")
        return cls(heads=heads, dim=dim, vdim=vdim, q_rank=_sized(m, "q_rank", where, required=True, minimum=1),
                   kv_rank=_sized(m, "kv_rank", where, required=True, minimum=1),
                   scale=take_float(m, "scale", required=True), window=_window(m, where))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "q_rank": self.q_rank,
                             "kv_rank": self.kv_rank, "scale": self.scale}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass
class FanitarDifferentialAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    rot_base: Optional[float] = None
    rot_dims: Optional[int] = None
    window: Optional[int] = None

    @classmethod
    def from_dict(cls, m: Dict[str, Any], where: str) -> "FanitarDifferentialAttention":
        heads = _sized(m, "heads", where, required=True, minimum=1)
        kv_heads = _sized(m, "kv_heads", where, default=heads, minimum=1)
        dim = _sized(m, "dim", where, required=True, minimum=1)
        vdim = _sized(m, "vdim", where, default=dim, minimum=1)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if max(2 * dim, vdim) > MAX_HEAD_DIM:       # the two maps of a key lie side by side in the cache
            raise ConfigError(f"config.json: {where}: two maps of {dim} and values of {vdim} are not served "
                              f"(up to {MAX_HEAD_DIM // 2} a map, values up to {MAX_HEAD_DIM})")
        rot = take_obj(m, "rot", where)
        base = dims = None
        if rot is not None:
            base = take_float(rot, "base", required=True, positive=True)
            dims = take_int(rot, "dims", required=True, minimum=0)
            if dims % 2 or dims > dim:
                raise ConfigError(f"config.json: {where}: {dims} rotated channels of a map of {dim} (even, at most the map)")
            if dims == 0:
                base = dims = None
        return cls(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=take_float(m, "scale", required=True),
                   diff=take_float(m, "diff", required=True), rot_base=base, rot_dims=dims, window=_window(m, where))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale, "diff": self.diff}
        if self.rot_dims is not None:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        return d


@dataclass
class FanitarLayer:
    type: str
    mixer: Union[FanitarLatentAttention, FanitarDifferentialAttention]
    ff: Optional[int] = None          # None: no feed-forward
    limit: Optional[float] = None
    mlp_kind: str = "dense"

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": self.mlp_kind, "ff": self.ff, "limit": self.limit}}


@dataclass
class FanitarLoop:
    start: int
    stop: int
    times: int

    def to_dict(self) -> Dict[str, int]:
        return {"start": self.start, "stop": self.stop, "times": self.times}


MIXERS = {"latent_attention": FanitarLatentAttention, "attention": FanitarDifferentialAttention}
MLP_KINDS = ("dense",)


@dataclass
class FanitarConfig(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    layers: List[FanitarLayer] = field(default_factory=list)
    loop: Optional[FanitarLoop] = None
    eos_token_ids: List[int] = field(default_factory=list)
    max_position_embeddings: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "FanitarConfig":
        norm = take_obj(d, "norm", "the model", required=True)
        entries = d.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[FanitarLayer] = []
        for i, e in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}: no mixer of type {kind!r}; there are {sorted(MIXERS)}")
            mixer = MIXERS[kind].from_dict(take_obj(e, "mixer", where, required=True), where)
            mlp = take_obj(e, "mlp", where)
            ff = limit = None
            mlp_kind = "dense"
            if mlp is not None:
                mlp_kind = mlp.get("kind", "dense")
                if mlp_kind not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}: no feed-forward of kind {mlp_kind!r}; there are {MLP_KINDS}")
                ff = take_int(mlp, "ff", required=True, minimum=1)
                limit = take_float(mlp, "limit", required=True, positive=True)
            layers.append(FanitarLayer(type=kind, mixer=mixer, ff=ff, limit=limit, mlp_kind=mlp_kind))
        loop = None
        lp = take_obj(d, "loop", "the model")
        if lp is not None:
            loop = FanitarLoop(start=take_int(lp, "start", required=True, minimum=0),
                               stop=take_int(lp, "stop", required=True, minimum=0),
                               times=take_int(lp, "times", required=True, minimum=1))
            if not (loop.start < loop.stop <= len(layers)):
                raise ConfigError(f"config.json: loop over layers {loop.start} .. {loop.stop - 1} of {len(layers)}")
        emb = take_obj(d, "embedding", "the model")
        known = {"architecture", "architectures", "vocab", "width", "norm", "layers", "loop", "embedding", "logit_scale",
                 "eos_token_id", "max_position_embeddings", "torch_dtype"}
        eos = d.get("eos_token_id")
        eos_ids = [eos] if isinstance(eos, int) and not isinstance(eos, bool) else list(eos or [])
        return cls(architecture=NAME, extra={k: v for k, v in d.items() if k not in known},
                   vocab_size=take_int(d, "vocab", required=True, minimum=1),
                   hidden_size=take_int(d, "width", required=True, minimum=1),
                   norm_eps=take_float(norm, "eps", required=True, positive=True),
                   embedding_scale=take_float(emb, "scale", default=1.0) if emb is not None else 1.0,
                   logit_scale=take_float(d, "logit_scale", default=1.0), layers=layers, loop=loop,
                   eos_token_ids=eos_ids,
                   max_position_embeddings=take_int(d, "max_position_embeddings", default=None, allow_none=True,
                                                    minimum=1))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": NAME, "vocab": self.vocab_size, "width": self.hidden_size,
                             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                             "logit_scale": self.logit_scale, "layers": [l.to_dict() for l in self.layers]}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        d.update(self.extra)
        return d
