"""A plain, slow implementation of the Sozetar design in float64 on the CPU, written
from its equations, one function per mechanism.  It shares no code with the package:
it reads a configuration as a plain dict and weights as a dict of tensors by name.

Notation: x [n, width] is the residual stream of one sequence, position p = row index.

  layer:      x <- x + LN(mixer(x));  x <- x + LN(ffn(x))   (the second only with a feed-forward)
  LN(t)     = (t - mean t) / sqrt(mean (t - mean t)^2 + eps) * w
  mixer(h):   q = rmsw(Wq h + bq; wq) * temp(p),  k = rmsw(Wk h + bk; wk),  v = Wv h + bv
              rmsw(t; w) = t / sqrt(mean t^2 + eps) * w  over ALL channels of the projection
              temp(p)  = 1 + coef * ln(floor((p + 1) / every) + 1)
              s_h(p, j) = scale * q_h(p) . k_g(j) - slope_h * (p - j),  slope_h = 2^(-8 (h + 1) / H)
              j visible from p iff 0 <= p - j < window
              a_h(p, j) = exp(s) / (exp(sink_h) + sum_visible exp(s))
              out_h(p) = sigmoid(Wg h)_h * sum_j a_h(p, j) v_g(j);   result = Wo concat_h out_h + bo
  ffn(h)    = Wd (gelu_tanh(Wg h) * (Wu h))
  logits    = head LN(x)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def widen(weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(F) if v.dtype.is_floating_point else v) for k, v in weights.items()}


def layer_norm(t: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mean = t.mean(-1, keepdim=True)
    dev = t - mean
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * w


def rms_over_projection(t: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """t [n, channels of all heads]: one root mean square per row."""
    return t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w


def query_temperature(n: int, coef: float, every: float) -> torch.Tensor:
    p = torch.arange(n, dtype=F)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def head_slopes(heads: int) -> torch.Tensor:
    h = torch.arange(1, heads + 1, dtype=F)
    return torch.pow(torch.tensor(2.0, dtype=F), -8.0 * h / heads)


def visible(n: int, window: Optional[int]) -> torch.Tensor:
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    return ok


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, slopes: Optional[torch.Tensor],
           sinks: Optional[torch.Tensor], window: Optional[int], first_row: int = 0) -> torch.Tensor:
    """q [n, H, dk], k [n, G, dk], v [n, G, dv] -> [n, H, dv].  Row by row and key by key.  Rows before
    `first_row` are left zero (a caller that asks for the last rows only)."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        for p in range(first_row, n):
            lo = 0 if window is None else max(0, p - window + 1)
            s = (k[lo:p + 1, g] @ q[p, h]) * scale
            if slopes is not None:
                s = s - slopes[h] * (p - torch.arange(lo, p + 1, dtype=F))
            top = s.max() if sinks is None else torch.maximum(s.max(), sinks[h])
            e = torch.exp(s - top)
            den = e.sum() + (torch.exp(sinks[h] - top) if sinks is not None else 0.0)
            out[p, h] = (e / den) @ v[lo:p + 1, g]
    return out


def attention_mixer(W, prefix: str, m: dict, eps: float, h: torch.Tensor, kv_of_layer: dict, index: int) -> torch.Tensor:
    n = h.shape[0]
    H, G, dk = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    dv = m.get("vdim", dk)
    q = rms_over_projection(h @ W[prefix + "q"].T + W[prefix + "q.b"], W[prefix + "q.norm"], eps)
    if m.get("kv_from") is None:
        k = rms_over_projection(h @ W[prefix + "k"].T + W[prefix + "k.b"], W[prefix + "k.norm"], eps)
        v = h @ W[prefix + "v"].T + W[prefix + "v.b"]
        kv_of_layer[index] = (k, v)
    else:
        k, v = kv_of_layer[m["kv_from"]]
    if m.get("q_temp"):
        q = q * query_temperature(n, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    window = m["mask"]["size"] if m.get("mask") else None
    o = attend(q.view(n, H, dk), k.view(n, G, dk), v.view(n, G, dv), m["scale"], head_slopes(H),
               W[prefix + "sink"], window)
    o = o * torch.sigmoid(h @ W[prefix + "g"].T)[:, :, None]
    return o.reshape(n, H * dv) @ W[prefix + "o"].T + W[prefix + "o.b"]


def gated_ffn(W, prefix: str, h: torch.Tensor) -> torch.Tensor:
    return (gelu_tanh(h @ W[prefix + "gate"].T) * (h @ W[prefix + "up"].T)) @ W[prefix + "down"].T


def forward(weights: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence, every position.  `streams`: receives x after each layer."""
    W = widen(weights)
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)]
    kv_of_layer: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        assert layer["type"] == "attention"
        x = x + layer_norm(attention_mixer(W, f"l{i}.mix.", layer["mixer"], eps, x, kv_of_layer, i), W[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + layer_norm(gated_ffn(W, f"l{i}.mlp.", x), W[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ W["head"].T


def generate_greedy(weights, cfg: dict, prompt: List[int], n_new: int):
    """Greedy continuation by running the whole sequence again for every token; of equal maxima
    the last (as the package's sampler)."""
    ids, out = list(prompt), []
    for _ in range(n_new):
        lg = forward(weights, cfg, ids)[-1]
        top = lg.max()
        t = int(torch.nonzero(lg == top).max())
        out.append(t)
        ids.append(t)
    return out


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model of this configuration, by name."""
    Wd, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, Wd)}
    for i, layer in enumerate(cfg["layers"]):
        m = layer["mixer"]
        H, G, dk = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
        dv = m.get("vdim", dk)
        p = f"l{i}."
        out[p + "norm1"] = (Wd,)
        out[p + "mix.q"], out[p + "mix.q.b"], out[p + "mix.q.norm"] = (H * dk, Wd), (H * dk,), (H * dk,)
        if m.get("kv_from") is None:
            out[p + "mix.k"], out[p + "mix.k.b"], out[p + "mix.k.norm"] = (G * dk, Wd), (G * dk,), (G * dk,)
            out[p + "mix.v"], out[p + "mix.v.b"] = (G * dv, Wd), (G * dv,)
        out[p + "mix.sink"], out[p + "mix.g"] = (H,), (H, Wd)
        out[p + "mix.o"], out[p + "mix.o.b"] = (Wd, H * dv), (Wd,)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out[p + "norm2"] = (Wd,)
            out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = (ff, Wd), (ff, Wd), (Wd, ff)
    out["final.norm"], out["head"] = (Wd,), (V, Wd)
    return out


def random_weights(cfg: dict, seed: int, std: float = 0.3, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Weights of the test's own making: matrices and biases N(0, std), norm weights around 1,
    sinks N(0, 1), all rounded to `dtype` (what a model file would hold)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        t = torch.randn(shape, generator=g, dtype=torch.float32)
        if name.endswith(("norm1", "norm2", ".norm")):
            t = 1.0 + 0.2 * t
        elif name.endswith("sink"):
            pass
        else:
            t = std * t
        out[name] = t.to(dtype)
    return out
