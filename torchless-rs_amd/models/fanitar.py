"""Fanitar as a list of parts.

A decoder-only model whose layers norm on both sides of a sublayer (`sandwich_norm` block,
RMS norms), whose mixers are attention out of latents (`latent_attention`: a sliding window, a
sink, a gate per channel) and differential attention (`differential_attention`: two maps a
head, biases, a rotation of part of each map, grouped KV heads), whose feed-forward is gated
with a clamped swish (`swish_clamped` with alpha 1.702 and a shift of 1 on the up branch) and
whose embedding and logits carry a factor each.  A run of layers may be gone through several
times with the same weights and a cache of its own each time; before each pass the stream
receives a learned vector and, from the second pass on, the embedding's output again
(`pass_entry`).  Tensor names: `embed`, `loop.step`, `l<i>.norm1`, `norm1b`, `norm2`, `norm2b`,
`l<i>.mix.*`, `l<i>.mlp.{gate,up,down}`, `final.norm`, `head`.  Every size comes from the
configuration, layer by layer.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.fanitar import NAME, FanitarConfig, FanitarLatentAttention
from ..parts.base import LayerSpec, ModelSpec, PartSpec, Run

SWISH_ALPHA = 1.702         # the gate of the feed-forward: g * logistic(1.702 g)
UP_SHIFT = 1.0              # ... times (up + 1)


def fanitar_spec(cfg: FanitarConfig) -> ModelSpec:
    H = cfg.hidden_size
    norm = PartSpec("rmsnorm", {"size": H, "eps": cfg.norm_eps, "name": ""})     # the tensor is the prefix itself
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, FanitarLatentAttention):
            mixer = PartSpec("latent_attention", {
                "hidden_size": H, "n_heads": m.heads, "head_dim": m.dim, "v_head_dim": m.vdim, "q_rank": m.q_rank,
                "kv_rank": m.kv_rank, "scale": m.scale, "norm_eps": cfg.norm_eps, "window": m.window, "sink": True,
                "gate": True, "prefix": "mix."})
        else:
            position = (PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims})
                        if m.rot_dims is not None else PartSpec("none"))
            mixer = PartSpec("differential_attention", {
                "hidden_size": H, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim,
                "lambda_init": m.diff, "norm_eps": cfg.norm_eps, "position": position, "scale": m.scale, "bias": True,
                "window": m.window, "prefix": "mix."})
        ffn = None
        if layer.ff is not None:
            ffn = PartSpec("gated", {"hidden_size": H, "intermediate_size": layer.ff, "prefix": "mlp.",
                                     "activation": "swish_clamped",
                                     "activation_constants": {"alpha": SWISH_ALPHA, "limit": layer.limit, "shift": UP_SHIFT},
                                     "names": {"gate": "gate", "up": "up", "down": "down"}})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, ffn=ffn, mixer_norm=norm, mixer_out_norm=norm,
                                ffn_norm=norm if ffn is not None else None,
                                ffn_out_norm=norm if ffn is not None else None,
                                block=PartSpec("sandwich_norm", {"names": ("norm1", "norm1b", "norm2", "norm2b")})))
    n = len(layers)
    stream_parts = []
    if cfg.loop is None:
        schedule = [Run(i) for i in range(n)]
    else:
        lp = cfg.loop
        stream_parts.append(("loop.", PartSpec("pass_entry", {"hidden_size": H, "passes": lp.times, "name": "step"})))
        schedule = [Run(i) for i in range(lp.start)]
        for t in range(lp.times):
            schedule += [Run(i, entry=(0, t) if i == lp.start else None) for i in range(lp.start, lp.stop)]
        schedule += [Run(i) for i in range(lp.stop, n)]
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "embed",
                                      "scale": cfg.embedding_scale}),
        embedding_prefix="",
        layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "head",
                                 "scale": cfg.logit_scale}),
        head_prefix="", stream_parts=stream_parts,
    )


register_architecture(NAME, FanitarConfig, fanitar_spec)
