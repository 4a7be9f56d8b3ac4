"""A plain, slow implementation of Fanitar in float64, one function per mechanism, written
from the design's equations.  It shares no code with the package: the tests compare the
engine against it.

Notation.  x: the residual stream [T, W].  rms(t, w) = t / sqrt(mean(t^2) + eps) * w over the
last axis (w left out: no weight).  A layer is
    x <- x + rms(mixer(rms(x, n1)), n1b);  x <- x + rms(ff(rms(x, n2)), n2b)    (the second only with a feed-forward).
Layers a .. b-1 may be repeated R times with the same weights; before repetition t the stream
receives the vector step[t] and, for t > 0, the embedding's output e once more.
"""
import math

import torch

F64 = torch.float64


def rms(t, eps, w=None):
    y = t / torch.sqrt((t * t).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def visible(T, window=None):
    """[T, T] bool: row p sees column j iff j <= p and (with a window) p - j < window."""
    p = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= p
    if window:
        ok &= (p - j) < window
    return ok


def softmax_with_sink(s, ok, sink=None):
    """s [..., T, T] scores, ok [T, T]; `sink` [...] adds exp(sink) to the denominator only."""
    s = s.masked_fill(~ok, -math.inf)
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[..., None, None].expand_as(m))
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[..., None, None] - m)
    return e / den


def latent_attention(h, w, p, m, eps):
    """h [T, W]; tensors w[p + ...]; m: the mixer's entry of the configuration."""
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    cq = rms(h @ w[p + "dq"].T, eps, w[p + "dq.norm"])
    c = rms(h @ w[p + "dkv"].T, eps, w[p + "dkv.norm"])
    q = (cq @ w[p + "uq"].T).view(T, H, d).transpose(0, 1)          # [H, T, d]
    k = (c @ w[p + "uk"].T).view(T, H, d).transpose(0, 1)
    v = (c @ w[p + "uv"].T).view(T, H, dv).transpose(0, 1)
    s = (q @ k.transpose(1, 2)) * m["scale"]
    a = softmax_with_sink(s, visible(T, (m.get("mask") or {}).get("size")), w[p + "sink"])
    heads = (a @ v).transpose(0, 1).reshape(T, H * dv)
    heads = heads * torch.sigmoid(h @ w[p + "g"].T)
    return heads @ w[p + "o"].T


def rotate(t, positions, base, dims):
    """t [T, n, d]: the first `dims` channels of every unit, pair (i, i + dims/2) turned by
    positions * base^(-2i/dims)."""
    if not dims:
        return t
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = positions.to(F64)[:, None] * f[None, :]
    co, si = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = t[..., :half], t[..., half:dims]
    return torch.cat([a * co - b * si, b * co + a * si, t[..., dims:]], dim=-1)


def diff_lambda(w, p, init):
    return float(torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + init)


def differential_attention(h, w, p, m, eps):
    T, H, G, d, dv = h.shape[0], m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    q = rotate((h @ w[p + "q"].T + w[p + "q.b"]).view(T, 2 * H, d), pos, rot.get("base"), rot.get("dims"))
    k = rotate((h @ w[p + "k"].T + w[p + "k.b"]).view(T, 2 * G, d), pos, rot.get("base"), rot.get("dims"))
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    ok = visible(T, (m.get("mask") or {}).get("size"))
    lam = diff_lambda(w, p, m["diff"])
    out = torch.empty(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        maps = []
        for mp in range(2):
            s = (q[:, 2 * hd + mp] @ k[:, 2 * g + mp].T) * m["scale"]
            maps.append(softmax_with_sink(s, ok) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hd] = rms(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ w[p + "o"].T


def clamped_feed_forward(h, w, p, m):
    lim = m["limit"]
    g = torch.clamp(h @ w[p + "gate"].T, max=lim)
    u = torch.clamp(h @ w[p + "up"].T, min=-lim, max=lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def layer(x, w, cfg, i):
    L, p, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h = rms(x, eps, w[p + "norm1"])
    if L["type"] == "latent_attention":
        y = latent_attention(h, w, p + "mix.", L["mixer"], eps)
    else:
        y = differential_attention(h, w, p + "mix.", L["mixer"], eps)
    x = x + rms(y, eps, w[p + "norm1b"])
    if L.get("mlp") is not None:
        x = x + rms(clamped_feed_forward(rms(x, eps, w[p + "norm2"]), w, p + "mlp.", L["mlp"]), eps, w[p + "norm2b"])
    return x


def order_of_runs(cfg):
    """[(layer, t or None)]: t is set on the first layer of repetition t."""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        runs += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, None) for i in range(lp["stop"], n)]


def forward(weights, cfg, ids, streams=None):
    """float64 logits [T, vocab]; `streams` (a list) receives x after every run of a layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    e = w["embed"][torch.tensor(ids)] * cfg.get("embedding", {}).get("scale", 1.0)
    x = e
    for i, t in order_of_runs(cfg):
        if t is not None:
            if t > 0:
                x = x + e
            x = x + w["loop.step"][t]
        x = layer(x, w, cfg, i)
        if streams is not None:
            streams.append(x.clone())
    return rms(x, cfg["norm"]["eps"], w["final.norm"]) @ w["head"].T * cfg.get("logit_scale", 1.0)


def generate_greedy(weights, cfg, ids, n):
    ids, out = list(ids), []
    for _ in range(n):
        t = int(forward(weights, cfg, ids)[-1].argmax())
        out.append(t)
        ids.append(t)
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16):
    """Every tensor of a model of `cfg`, drawn from `seed` (bfloat16 as the files hold them).  Queries and
    keys get a gain of 1.3: scores of a few units, so that the softmax is far from uniform and yet a
    rounding of q or k to 8 bits (a share 2^-9 of a score) moves a weight by less than a hundredth."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    out = {}

    def mat(name, rows, cols, gain=1.0):
        out[name] = (torch.randn(rows, cols, generator=g) * gain / math.sqrt(cols)).to(dtype)

    def vec(name, n, mean=0.0, std=1.0):
        out[name] = (mean + std * torch.randn(n, generator=g)).to(dtype)

    out["embed"] = (torch.randn(cfg["vocab"], W, generator=g) * 0.5).to(dtype)
    if cfg.get("loop"):
        out["loop.step"] = (torch.randn(cfg["loop"]["times"], W, generator=g) * 0.5).to(dtype)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        names = ["norm1", "norm1b"] + (["norm2", "norm2b"] if L.get("mlp") is not None else [])
        for nm in names:
            vec(p + nm, W, 1.0, 0.2)
        d, dv = m["dim"], m.get("vdim", m["dim"])
        if L["type"] == "latent_attention":
            H = m["heads"]
            mat(p + "mix.dq", m["q_rank"], W)
            vec(p + "mix.dq.norm", m["q_rank"], 1.0, 0.2)
            mat(p + "mix.uq", H * d, m["q_rank"], 1.3)
            mat(p + "mix.dkv", m["kv_rank"], W)
            vec(p + "mix.dkv.norm", m["kv_rank"], 1.0, 0.2)
            mat(p + "mix.uk", H * d, m["kv_rank"], 1.3)
            mat(p + "mix.uv", H * dv, m["kv_rank"])
            vec(p + "mix.sink", H, 0.0, 1.0)
            mat(p + "mix.g", H * dv, W, 2.0)
            mat(p + "mix.o", W, H * dv)
        else:
            H, G = m["heads"], m.get("kv_heads", m["heads"])
            mat(p + "mix.q", 2 * H * d, W, 1.3)
            vec(p + "mix.q.b", 2 * H * d, 0.0, 0.3)
            mat(p + "mix.k", 2 * G * d, W, 1.3)
            vec(p + "mix.k.b", 2 * G * d, 0.0, 0.3)
            mat(p + "mix.v", G * dv, W)
            vec(p + "mix.v.b", G * dv, 0.0, 0.3)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + "mix." + nm, d, 0.0, 0.3 / math.sqrt(d))
            mat(p + "mix.o", W, H * dv)
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            mat(p + "mlp.gate", ff, W, 1.5)
            mat(p + "mlp.up", ff, W, 1.5)
            mat(p + "mlp.down", W, ff)
    vec("final.norm", W, 1.0, 0.2)
    mat("head", cfg["vocab"], W)
    return out
