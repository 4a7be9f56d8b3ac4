"""Sozetar as a list of parts.

A decoder-only model whose layers norm a sublayer's OUTPUT before the residual sum
(`output_norm` block, layer norm with a weight and no bias), whose mixer is the
attention with score terms (`scored_attention`: biases, a norm of q and k over the
whole projection, a factor on q that grows with the position, a distance bias with
slopes 2^(-8 (h + 1) / heads), a sliding window, a sink, a gate per head, values of
their own width, and layers that read an earlier layer's keys and values) and whose
feed-forward is gated with the tanh form of gelu.  Tensor names: `embed`,
`l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.{gate,up,down}`, `final.norm`,
`head`.  Every size comes from the configuration, layer by layer.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.sozetar import NAME, SozetarConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, Run

SLOPE_EXPONENT = 8.0        # slope of head h: 2^(-8 (h + 1) / heads)


def sozetar_spec(cfg: SozetarConfig) -> ModelSpec:
    H = cfg.hidden_size
    norm = PartSpec("layernorm", {"size": H, "eps": cfg.norm_eps, "name": ""})     # the tensor is the prefix itself
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        mixer = PartSpec("scored_attention", {
            "hidden_size": H, "n_heads": m.heads, "n_kv_heads": m.kv_heads, "head_dim": m.dim,
            "v_head_dim": m.vdim, "window": m.window, "own_kv": m.kv_from is None, "scale": m.scale,
            "bias": True, "qk_norm_eps": cfg.norm_eps,
            "q_temperature": None if m.q_temp_coef is None else (m.q_temp_coef, m.q_temp_every),
            "distance_slope_exponent": SLOPE_EXPONENT, "sink": True, "head_gate": True, "prefix": "mix."})
        ffn = None
        if layer.ff is not None:
            ffn = PartSpec("gated", {"hidden_size": H, "intermediate_size": layer.ff, "prefix": "mlp.",
                                     "activation": "gelu_tanh",
                                     "names": {"gate": "gate", "up": "up", "down": "down"}})
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, ffn=ffn, mixer_norm=norm,
                                ffn_norm=norm if ffn is not None else None,
                                block=PartSpec("output_norm", {"mixer_norm_name": "norm1", "ffn_norm_name": "norm2"})))
        schedule.append(Run(i, kv_from=m.kv_from))
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "embed"}),
        embedding_prefix="",
        layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "name": "head"}),
        head_prefix="",
    )


register_architecture(NAME, SozetarConfig, sozetar_spec)
