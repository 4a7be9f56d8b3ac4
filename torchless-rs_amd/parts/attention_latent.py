"""Attention whose queries, keys and values come out of low-rank latents.

With h the mixer's input, rms(t) = t / sqrt(mean(t^2) + eps) and H heads:

    c_q = rms(W_dq h) * w_q          q_h = W_uq[h] c_q            (q_rank channels between)
    c   = rms(W_dkv h) * w_c         k_h = W_uk[h] c ,  v_h = W_uv[h] c    (kv_rank channels)
    s_h(p, j) = (q_h(p) . k_h(j)) * scale        over the visible keys (causal, optional window)
    out = W_o ( concat_h(softmax(s_h) v_h) * logistic(W_g h) )

No rotation.  Optional: a sliding window; a sink, a learned score per head without key or value
that counts once in the softmax's denominator (`sink`); the gate per CHANNEL of the concatenated
heads (`gate`).  The three down projections that read h (to c_q, to c, and the gate) are one
product; one row-wise kernel norms both latents and applies the logistic function; the up
projections of keys and values are one product as well.

The cache keeps k and v per head, as the framework's attention kernels read them (keys [64][d],
values transposed, a page of 64 positions): expanding c once per token at the time it is
written, not once per query that looks back at it.  The window bounds what a sequence holds.
Scores, softmax weights, both norms and the gate's function are float32 in both dtypes.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.cache import KVRequest
from ..kernels import ops
from ..weights.binding import WeightSpec
from .attention_scored import attend_and_commit
from .base import Mixer, flush_pending, register_part
from .linear import Linear


class LatentAttentionMixer(Mixer):
    graph_safe = True

    NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
             "sink": "sink", "gate": "g", "o": "o"}

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, v_head_dim: int, q_rank: int, kv_rank: int,
                 scale: float, norm_eps: float, window: Optional[int] = None, sink: bool = False, gate: bool = False,
                 prefix: str = "mix.", names: Optional[Dict[str, str]] = None):
        unknown = set(names or {}) - set(self.NAMES)
        if unknown:
            raise ValueError(f"latent attention: no tensors called {sorted(unknown)}; there are {sorted(self.NAMES)}")
        self.names = dict(self.NAMES, **(names or {}))
        self.H, self.nq, self.dk, self.dv = int(hidden_size), int(n_heads), int(head_dim), int(v_head_dim)
        self.qr, self.kvr = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(norm_eps)
        self.window = int(window) if window else None
        self.sink, self.gate = bool(sink), bool(gate)
        self.ng = self.nq * self.dv if self.gate else 0
        self.prefix = prefix
        self.down = self.uq = self.ukv = self.o = None

    def kv_request(self):
        return KVRequest(self.nq, self.dk, self.window, None if self.dv == self.dk else self.dv)

    def kv_reach(self):
        return self.window

    def may_capture(self, n_rows: int) -> bool:
        return self.down is not None and all(l.own_kernels(n_rows) for l in (self.down, self.uq, self.ukv, self.o))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, nm = self.prefix, self.names
        out = {p + nm["dq"]: WeightSpec((self.qr, self.H)), p + nm["dq_norm"]: WeightSpec((self.qr,), init="ones"),
               p + nm["uq"]: WeightSpec((self.nq * self.dk, self.qr)),
               p + nm["dkv"]: WeightSpec((self.kvr, self.H)), p + nm["dkv_norm"]: WeightSpec((self.kvr,), init="ones"),
               p + nm["uk"]: WeightSpec((self.nq * self.dk, self.kvr)),
               p + nm["uv"]: WeightSpec((self.nq * self.dv, self.kvr))}
        if self.sink:
            out[p + nm["sink"]] = WeightSpec((self.nq,))
        if self.gate:
            out[p + nm["gate"]] = WeightSpec((self.ng, self.H))
        out[p + nm["o"]] = WeightSpec((self.H, self.nq * self.dv))
        return out

    def load(self, tensors, compute_dtype) -> None:
        p, nm = self.prefix, self.names

        def t(key):
            return tensors[p + nm[key]]

        def fused(keys):
            ws = [t(k) for k in keys]
            if len({w.dtype for w in ws}) > 1:
                ws = [w.to(torch.float32) for w in ws]
            return torch.cat(ws, dim=0)

        self.down = Linear(fused(["dq", "dkv"] + (["gate"] if self.gate else [])), tiled=True)
        self.uq = Linear(t("uq"), tiled=True)
        self.ukv = Linear(fused(["uk", "uv"]), tiled=True)
        self.o = Linear(t("o"), tiled=True)
        self.wq = t("dq_norm").to(torch.float32).contiguous()
        self.wc = t("dkv_norm").to(torch.float32).contiguous()
        sinks = t("sink").to(torch.float32).contiguous() if self.sink else None
        self.terms = ops.ScoreTerms(self.scale, self.window, None, sinks)

    def produce(self, ctx, run, y: torch.Tensor, out: torch.Tensor):
        n, nq, dk, dv, ng = y.shape[0], self.nq, self.dk, self.dv, self.ng
        ws = ctx.workspace
        proj = ws.get("lat_proj", (n, self.qr + self.kvr + ng), torch.float32)
        self.down(y, proj)
        cq = ws.get("lat_cq", (n, self.qr), ctx.dtype)
        c = ws.get("lat_c", (n, self.kvr), ctx.dtype)
        gate = ws.get("lat_gate", (n, ng), torch.float32) if ng else None
        ops.latent_norms(proj, self.qr, self.kvr, self.wq, self.wc, self.eps, cq, c, gate)
        qf = ws.get("lat_qf", (n, nq * dk), torch.float32)
        self.uq(cq, qf)
        kvf = ws.get("lat_kvf", (n, nq * (dk + dv)), torch.float32)
        self.ukv(c, kvf)
        q = ws.get("lat_q", (n, nq, dk), ctx.dtype)
        att = ws.get("lat_att", (n, nq, dv), ctx.dtype)
        if ctx.all_single:      # one token a sequence: k and v go straight into the pages
            group = run.kv_group
            ops.split_heads(qf, kvf, ctx.row_pos, nq, nq, dk, dv, q, None, None, table=ctx.tables[run.kv_group_index],
                            ring_pages=group.ring_pages, pages=group.storage[run.kv_layer])
            k = v = None
        else:
            k = ws.get("lat_k", (n, nq, dk), ctx.dtype)
            v = ws.get("lat_v", (n, nq, dv), ctx.dtype)
            ops.split_heads(qf, kvf, ctx.row_pos, nq, nq, dk, dv, q, k, v)
        attend_and_commit(ctx, run, q, k, v, nq, dk, dv, self.terms, None, att)
        if gate is not None:
            ops.mul_gate(att, gate)
        self.o(att.view(n, nq * dv), out)
        return None

    def forward(self, ctx, run, y: torch.Tensor, x: torch.Tensor) -> None:
        flush_pending(ctx, x)
        z = ctx.workspace.get("lat_z", tuple(x.shape), torch.float32)
        self.produce(ctx, run, y, z)
        ops.add_partials(x, z.view(1, *z.shape))


register_part("mixer", "latent_attention", LatentAttentionMixer)
