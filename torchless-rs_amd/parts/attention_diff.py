"""Differential attention: two attention maps per head over the same values, subtracted.

H query heads over G key/value heads (head h reads KV head h // (H / G)); per head TWO
queries and per KV head TWO keys of d channels each (map 1, map 2) and one value of dv:

    s_m(p, j) = (q_m(p) . k_m(j)) * scale ,  a_m = softmax_j(s_m) v         m = 1, 2
    o = a_1 - lambda * a_2 ,   head = o / sqrt(mean(o^2) + eps) * (1 - lambda_init)
    lambda = exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + lambda_init       (one number a layer)

then the output projection over the concatenated heads.  Optional biases on q, k and v; the
position part rotates every MAP of q and k (its first `rotary_dim` channels).  Causal, with an
optional window.

The maps run through the framework's attention kernels unchanged: the cache keeps one key
of 2d channels per KV head and position, [map 1 | map 2], and a query of map m becomes a head
of 2d channels with its own channels in half m and zeros in the other half, so that the
product with the key is q_m . k_m exactly, the two maps of a head are two heads of the same
group, and both read the same values once.  (The price is twice the multiplications in the
score product; the value product and all memory traffic are what two maps need.)
lambda is worked out once at load, in float32; the difference and its norm are float32 (of maps
that the matrix-core kernels have rounded to bfloat16, or of the unrounded maps where the kernel that
sums in float runs: head sizes the matrix cores do not take, and the 32-bit path).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..cache.cache import KVRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .attention_scored import attend_and_commit
from .base import Mixer, PartSpec, flush_pending, make_part, register_part
from .linear import Linear


class DifferentialAttentionMixer(Mixer):
    graph_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
             "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, v_head_dim: int,
                 lambda_init: float, norm_eps: float, position: Optional[PartSpec] = None, scale: Optional[float] = None,
                 bias: bool = False, window: Optional[int] = None, prefix: str = "mix.",
                 names: Optional[Dict[str, str]] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"differential attention: {n_heads} heads are not a multiple of {n_kv_heads} KV heads")
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"differential attention: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.nq, self.nkv = int(hidden_size), int(n_heads), int(n_kv_heads)
        self.d, self.dv = int(head_dim), int(v_head_dim)
        self.lambda_init, self.eps = float(lambda_init), float(norm_eps)
        self.position = make_part("position", position if position is not None else PartSpec("none"))
        self.scale = 1.0 / math.sqrt(self.d) if scale is None else float(scale)
        self.bias = bool(bias)
        self.window = int(window) if window else None
        self.prefix = prefix
        self.proj = self.o = self.proj_bias = None
        self.lam = None

    def kv_request(self):
        return KVRequest(self.nkv, 2 * self.d, self.window, None if self.dv == 2 * self.d else self.dv)

    def kv_reach(self):
        return self.window

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows) and self.o.own_kernels(n_rows)

    def prefers_eager(self, n_new, len_before, device) -> bool:
        # few rows over a long context: the host cuts the keys into runs for workgroups of their own
        return (self.proj is not None and self.dv == 2 * self.d and ops.prefill_serves(self.proj.weight.dtype, self.dv)
                and ops.prefill_layout(n_new, len_before, self.window, 2 * self.nq, ops.compute_units(device)) is not None)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        Q, K, V = 2 * self.nq * self.d, 2 * self.nkv * self.d, self.nkv * self.dv
        out = {p + nm["q"]: WeightSpec((Q, self.H)), p + nm["k"]: WeightSpec((K, self.H)),
               p + nm["v"]: WeightSpec((V, self.H))}
        if self.bias:
            out.update({p + nm["q_bias"]: WeightSpec((Q,)), p + nm["k_bias"]: WeightSpec((K,)),
                        p + nm["v_bias"]: WeightSpec((V,))})
        for key in ("lq1", "lk1", "lq2", "lk2"):
            out[p + nm[key]] = WeightSpec((self.d,))
        out[p + nm["o"]] = WeightSpec((self.H, self.nq * self.dv))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names

        def t(key):
            return tensors[p + nm[key]]

        ws = [t("q"), t("k"), t("v")]
        if len({w.dtype for w in ws}) > 1:
            ws = [w.to(torch.float32) for w in ws]
        self.proj = Linear(torch.cat(ws, dim=0), tiled=True)
        self.o = Linear(t("o"), tiled=True)
        if self.bias:
            self.proj_bias = torch.cat([t(k).to(torch.float32) for k in ("q_bias", "k_bias", "v_bias")]).contiguous()
        f = {k: t(k).to(torch.float32) for k in ("lq1", "lk1", "lq2", "lk2")}
        lam = torch.exp((f["lq1"] * f["lk1"]).sum()) - torch.exp((f["lq2"] * f["lk2"]).sum()) + self.lambda_init
        self.lam = float(lam.to(torch.float32).item())
        self.terms = ops.ScoreTerms(self.scale, self.window, None, None)

    def produce(self, ctx, run, y: torch.Tensor, out: torch.Tensor):
        n, H, G, d, dv = y.shape[0], self.nq, self.nkv, self.d, self.dv
        ws = ctx.workspace
        proj = ws.get("diff_proj", (n, 2 * H * d + 2 * G * d + G * dv), torch.float32)
        self.proj(y, proj)
        rotation = self.position.rotation(y.device) or ops.NO_ROTATION
        q = ws.get("diff_q", (n, 2 * H, 2 * d), ctx.dtype)
        # where the kernel that keeps its sums in float runs, the two maps stay unrounded until their difference
        cores = ops.scored_on_matrix_cores(ctx.dtype, 2 * d, dv)
        maps = ws.get("diff_maps", (n, 2 * H, dv), ctx.dtype if cores else torch.float32)
        if ctx.all_single:      # one token a sequence: k and v go straight into the pages
            group = run.kv_group
            ops.diff_split(proj, self.proj_bias, ctx.row_pos, rotation, H, G, d, dv, q, None, None,
                           table=ctx.tables[run.kv_group_index], ring_pages=group.ring_pages,
                           pages=group.storage[run.kv_layer])
            k = v = None
        else:
            k = ws.get("diff_k", (n, G, 2 * d), ctx.dtype)
            v = ws.get("diff_v", (n, G, dv), ctx.dtype)
            ops.diff_split(proj, self.proj_bias, ctx.row_pos, rotation, H, G, d, dv, q, k, v)
        attend_and_commit(ctx, run, q, k, v, G, 2 * d, dv, self.terms, None, maps)
        att = ws.get("diff_att", (n, H, dv), ctx.dtype)
        ops.diff_combine(maps, self.lam, self.eps, 1.0 - self.lambda_init, att)
        self.o(att.view(n, H * dv), out)
        return None

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        flush_pending(ctx, x)
        z = ctx.workspace.get("diff_z", tuple(x.shape), torch.float32)
        self.produce(ctx, run, y, z)
        ops.add_partials(x, z.view(1, *z.shape))


register_part("mixer", "differential_attention", DifferentialAttentionMixer)
