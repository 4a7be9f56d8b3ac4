"""Fanitar on the GPU against the plain implementation of `plain_fanitar.py`: every new kernel
alone, the two mixers' steps around the attention kernels with keys made to stand out, then whole
models of the tests' own sizes through the engine: whole prompts, the stream after every run of a
layer, decoding token by token, portions down to two tokens, unequal batches, slots and pages
used again, long decoding past windows and rings, and greedy generation through the entry point."""
import copy
import json
import os
import subprocess
import sys
import types

import numpy as np
import pytest
import torch

import plain_fanitar as plain
from test_fanitar_config import MIXED, diff, latent, layer
from test_gpu_sozetar import some_prompts, write_model
from util import rel_err, rms_err

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
RMS = {"float32": 1e-5, "bfloat16": 2.5e-2}

# heads that the matrix cores take (keys and values of 64; two maps of 32 beside values of 64), windows that
# are no multiple of a page, two passes from the first layer on
CORES = {"architecture": "Fanitar", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
         "logit_scale": 1.5, "loop": {"start": 0, "stop": 2, "times": 2}, "layers": [
             layer(latent(4, 64, 64, 48, 80, 0.125, window=100), ff=192, limit=1.2),
             layer(diff(4, 2, 32, 64, 0.18, 0.4, rot=(10000.0, 32)), ff=128, limit=0.9),
             layer(latent(2, 32, 32, 64, 32, 0.18, window=70), ff=64, limit=3.0),
         ]}
# what a model may happen to make 1 or equal: one head, one pass, a window of one (a position sees itself
# alone), of exactly one page, no rotation, a factor of 1 on embedding and logits (left out), the loop
# over every layer
ONES = {"architecture": "Fanitar", "vocab": 96, "width": 32, "norm": {"eps": 1e-4},
        "loop": {"start": 0, "stop": 3, "times": 1}, "layers": [
            layer(latent(1, 16, 16, 8, 8, 0.25, window=1), ff=32, limit=1.0),
            layer(diff(1, 1, 8, 16, 0.35, 0.5), ff=16, limit=1.0),
            layer(latent(2, 8, 8, 16, 16, 0.35, window=64)),
        ]}
# sizes that no kernel's fast way takes: a width that is no multiple of 8, odd ranks, heads of 12 and 20, three heads,
# an odd vocabulary, values narrower than the two maps together, no loop at all
ODD = {"architecture": "Fanitar", "vocab": 131, "width": 100, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.7},
       "logit_scale": 3.0, "layers": [
           layer(latent(3, 12, 20, 18, 27, 0.29, window=33), ff=50, limit=0.8),
           layer(diff(3, 3, 10, 12, 0.3, 0.4, rot=(300.0, 6), window=65), ff=36, limit=4.0),
           layer(diff(6, 2, 12, 20, 0.29, 0.2, rot=(20.0, 12))),
       ]}
# head sizes that the matrix cores take but that are none of 64, 128 and 256 (48 and 80 wide, keys of two maps of
# 24 and 40), three passes over the last two layers, a window of three pages and a bit
HEADS = {"architecture": "Fanitar", "vocab": 300, "width": 192, "norm": {"eps": 1e-5}, "embedding": {"scale": 12.0},
         "logit_scale": 0.8, "loop": {"start": 1, "stop": 3, "times": 3}, "layers": [
             layer(diff(6, 3, 24, 48, 0.2, 0.6, rot=(5000.0, 16)), ff=256, limit=2.0),
             layer(latent(3, 48, 48, 72, 56, 0.15, window=200), ff=160, limit=1.0),
             layer(diff(2, 1, 40, 80, 0.16, 0.45, rot=(100.0, 40)), ff=96, limit=6.0),
         ]}
CONFIGS = {"mixed": MIXED, "cores": CORES, "ones": ONES, "odd": ODD, "heads": HEADS}
LENGTHS = {"mixed": [1, 7, 23, 70], "cores": [5, 64, 129, 330], "ones": [2, 65, 130, 200], "odd": [4, 33, 67, 140],
           "heads": [3, 50, 131, 260]}
NAMES = list(CONFIGS)


def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype is not None else t.to("cuda")


# ---------------------------------------------------------------------------------------------
# the kernels one by one
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("H", [32, 100, 1030, 4096])
@pytest.mark.parametrize("out_dtype", DTYPES)
def test_the_norm_of_an_output_into_the_stream_and_the_next_norm_with_it(H, out_dtype):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(H)
    z, x = torch.randn(5, H, generator=g) * 3, torch.randn(5, H, generator=g)
    w, w2 = 1 + 0.3 * torch.randn(H, generator=g), 1 + 0.3 * torch.randn(H, generator=g)
    want = x.double() + plain.rms(z.double(), 1e-5, w.double())
    xs = dev(x.clone())
    ops.rmsnorm_add(dev(z), dev(w), 1e-5, xs)
    assert rel_err(xs, want) < 1e-6
    xs = dev(x.clone())
    out = torch.empty(5, H, dtype=TORCH[out_dtype], device="cuda")
    ops.rmsnorm_add(dev(z), dev(w), 1e-5, xs, dev(w2), 1e-3, out)
    assert rel_err(xs, want) < 1e-6
    assert rel_err(out, plain.rms(want, 1e-3, w2.double())) < (1e-5 if out_dtype == "float32" else 8e-3)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("limit, alpha, shift", [(0.7, 1.702, 1.0), (2.5, 1.0, 0.0)])
def test_the_clamped_gate(out_dtype, limit, alpha, shift):
    from torchless_rs_amd.kernels import ops
    gu = torch.randn(4, 2 * 50, generator=torch.Generator().manual_seed(1)) * 3
    out = torch.empty(4, 50, dtype=TORCH[out_dtype], device="cuda")
    ops.act_mul(dev(gu), out, "swish_clamped", {"alpha": alpha, "limit": limit, "shift": shift})
    g, u = gu[:, :50].double().clamp(max=limit), gu[:, 50:].double().clamp(-limit, limit)
    want = g * torch.sigmoid(alpha * g) * (u + shift)
    assert rel_err(out, want) < (1e-6 if out_dtype == "float32" else 8e-3)
    assert (gu[:, :50] > limit).any() and (gu[:, 50:] < -limit).any()
    with pytest.raises(ops.KernelError):
        ops.act_mul(dev(gu), out, "swish_clamped")
    with pytest.raises(ops.KernelError):
        ops.act_mul(dev(gu), out, "silu", {"limit": 1.0})


@pytest.mark.parametrize("K", [128, 192, 1024])           # the ring of LDS stages takes multiples of 128, whole rows of 512, the other kernel the rest
@pytest.mark.parametrize("M", [1, 8, 16, 17, 64, 100, 128, 300])
def test_the_clamped_gate_in_the_epilogue_of_the_product(K, M):
    """gate and up rows interleaved in blocks of 32: every kernel that a row count selects clamps its
    float sums and applies the gate itself; above the kernels' own rows the library's product is
    followed by the same function on bfloat16 pairs.  Two sets of constants one after the other: a
    launch takes the ones that were named with it."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.linear import interleave_pairs
    g = torch.Generator().manual_seed(M + K)
    I = 96
    a = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
    wg, wu = ((torch.randn(I, K, generator=g) * (4.0 / K ** 0.5)).to(torch.bfloat16) for _ in range(2))
    w = dev(interleave_pairs(wg, wu))
    gate, up = a.double() @ wg.double().T, a.double() @ wu.double().T
    for k in ({"alpha": 1.702, "limit": 0.9, "shift": 1.0}, {"alpha": 0.5, "limit": 3.0, "shift": -0.25}):
        out = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
        if M > ops.own_rows(K):
            gu = torch.empty(M, 2 * I, dtype=torch.bfloat16, device="cuda")
            ops.gemm_library(dev(a), w, gu)
            ops.silu_mul_pairs(gu, out, "swish_clamped", k)
        elif M > 16:
            ops.gemm_mid_bf16(dev(a), w, out, 1, silu_pair=True, pair_act=("swish_clamped", k))
        else:
            ops.gemm_bf16(dev(a), w, out, silu_pair=True, pair_act=("swish_clamped", k))
        gc, uc = gate.clamp(max=k["limit"]), up.clamp(-k["limit"], k["limit"])
        want = gc * torch.sigmoid(k["alpha"] * gc) * (uc + k["shift"])
        assert (gate > k["limit"]).any() and (up < -k["limit"]).any()
        assert rel_err(out, want) < (2e-2 if M > ops.own_rows(K) else 6e-3), k
    with pytest.raises(ops.KernelError):
        ops.gemm_bf16(dev(a[:1]), w, out[:1], silu_pair=True, pair_act="swish_clamped")


def test_factors_on_embedding_and_logits_and_the_entry_of_a_pass():
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    table = torch.randn(20, 24, generator=g).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32)
    out = torch.empty(4, 24, device="cuda")
    ops.embed(dev(table), dev(ids), out, 2.5)
    assert rel_err(out, table[ids.long()].double() * 2.5) < 1e-7
    x, e, v = torch.randn(4, 24, generator=g), torch.randn(4, 24, generator=g), torch.randn(24, generator=g)
    xs = dev(x.clone())
    ops.stream_entry(xs, None, dev(v))
    assert rel_err(xs, x.double() + v.double()) < 1e-7
    ops.stream_entry(xs, dev(e), dev(v))
    assert rel_err(xs, x.double() + 2 * v.double() + e.double()) < 1e-6
    ops.scale_(xs, 0.25)
    assert rel_err(xs, (x.double() + 2 * v.double() + e.double()) * 0.25) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("na, nb, ng", [(24, 40, 16), (18, 27, 60), (96, 96, 0), (1, 300, 7)])
def test_the_norms_of_the_latents_and_the_gate(dtype, na, nb, ng):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(na)
    proj = torch.randn(6, na + nb + ng, generator=g) * 2
    wa, wb = 1 + 0.2 * torch.randn(na, generator=g), 1 + 0.2 * torch.randn(nb, generator=g)
    a = torch.empty(6, na, dtype=TORCH[dtype], device="cuda")
    b = torch.empty(6, nb, dtype=TORCH[dtype], device="cuda")
    gate = torch.empty(6, ng, device="cuda") if ng else None
    ops.latent_norms(dev(proj), na, nb, dev(wa), dev(wb), 1e-3, a, b, gate)
    tol = 1e-6 if dtype == "float32" else 8e-3
    assert rel_err(a, plain.rms(proj[:, :na].double(), 1e-3, wa.double())) < tol
    assert rel_err(b, plain.rms(proj[:, na:na + nb].double(), 1e-3, wb.double())) < tol
    if ng:
        assert rel_err(gate, torch.sigmoid(proj[:, na + nb:].double())) < 1e-6
        x = torch.randn(6, ng, generator=g).to(TORCH[dtype])
        xs = dev(x.clone())
        ops.mul_gate(xs, gate)
        assert rel_err(xs, x.double() * torch.sigmoid(proj[:, na + nb:].double())) < tol


def pages_for_rows(dt, nkv, dk, dv, positions, seed):
    """A page table for single-token rows at `positions` (one sequence a row), pages dealt in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    n = len(positions)
    per = [p // 64 + 1 for p in positions]
    n_pages = sum(per) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    table = torch.zeros(n, max(per), dtype=torch.int32)
    for b in range(n):
        for i in range(per[b]):
            table[b, i] = order.pop()
    shape = (n_pages, 2, nkv, 64, dk) if dk == dv else (n_pages, nkv * 64 * (dk + dv))
    return dev(table), torch.zeros(shape, dtype=dt, device="cuda")


def read_page(pages, table, b, pos, nkv, dk, dv):
    """(k [nkv, dk], v [nkv, dv]) of sequence b's position `pos` as the pages hold them."""
    flat = pages[int(table[b, pos // 64])].reshape(-1)
    k = flat[:nkv * 64 * dk].view(nkv, 64, dk)[:, pos % 64]
    v = flat[nkv * 64 * dk:].view(nkv, dv, 64)[:, :, pos % 64]
    return k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, dk, dv", [(2, 16, 8), (3, 12, 20), (4, 64, 64)])
def test_the_split_into_heads_to_rows_and_to_pages(dtype, nq, dk, dv):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(dk)
    dt = TORCH[dtype]
    pos = [0, 63, 64, 200]
    qf, kvf = torch.randn(4, nq * dk, generator=g), torch.randn(4, nq * (dk + dv), generator=g)
    q, k, v = (torch.empty(4, nq, w, dtype=dt, device="cuda") for w in (dk, dk, dv))
    rp = dev(torch.tensor(pos, dtype=torch.int32))
    ops.split_heads(dev(qf), dev(kvf), rp, nq, nq, dk, dv, q, k, v)
    assert torch.equal(q.cpu(), qf.view(4, nq, dk).to(dt)) and torch.equal(k.cpu(), kvf[:, :nq * dk].reshape(4, nq, dk).to(dt))
    assert torch.equal(v.cpu(), kvf[:, nq * dk:].reshape(4, nq, dv).to(dt))
    table, pages = pages_for_rows(dt, nq, dk, dv, pos, 3)
    ops.split_heads(dev(qf), dev(kvf), rp, nq, nq, dk, dv, q, None, None, table=table, ring_pages=1 << 24, pages=pages)
    for b, p in enumerate(pos):
        pk, pv = read_page(pages, table.cpu(), b, p, nq, dk, dv)
        assert torch.equal(pk, k[b]) and torch.equal(pv, v[b])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, d, dv, dims, biased", [(4, 2, 8, 24, 4, True), (2, 2, 16, 32, 16, True), (3, 3, 10, 6, 6, False),
                                                        (6, 2, 12, 20, 0, True), (1, 1, 32, 64, 20, True)])
def test_the_split_of_a_differential_projection(dtype, H, G, d, dv, dims, biased):
    """Biases, the rotation of part of each map, the queries as heads of two maps' width with
    zeros in the other map's half, keys with both maps side by side, to rows and to pages."""
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(d)
    dt = TORCH[dtype]
    pos = [0, 5, 64, 1000]
    n, Q, K, V = 4, 2 * H * d, 2 * G * d, G * dv
    proj = torch.randn(n, Q + K + V, generator=g)
    bias = torch.randn(Q + K + V, generator=g) if biased else None
    base = 500.0
    rot = None
    if dims:
        f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
        rot = ops.Rotation(dev(f.float()), dims)
    q = torch.empty(n, 2 * H, 2 * d, dtype=dt, device="cuda")
    k = torch.empty(n, G, 2 * d, dtype=dt, device="cuda")
    v = torch.empty(n, G, dv, dtype=dt, device="cuda")
    rp = dev(torch.tensor(pos, dtype=torch.int32))
    ops.diff_split(dev(proj), dev(bias) if biased else None, rp, rot, H, G, d, dv, q, k, v)
    full = proj.double() + (bias.double() if biased else 0)
    p64 = torch.tensor(pos)
    wq = plain.rotate(full[:, :Q].reshape(n, 2 * H, d), p64, base, dims)
    wk = plain.rotate(full[:, Q:Q + K].reshape(n, 2 * G, d), p64, base, dims)
    tol = 2e-5 if dtype == "float32" else 8e-3        # float32: the angle of position 1000 carries 6e-5 of rounding
    qq = q.cpu().double().view(n, H, 2, 2, d)          # [head, map, half, channel]
    for m in range(2):
        assert rel_err(qq[:, :, m, m], wq.view(n, H, 2, d)[:, :, m]) < tol
        assert float(qq[:, :, m, 1 - m].abs().max()) == 0.0
    assert rel_err(k.view(n, 2 * G, d), wk) < tol
    assert rel_err(v.view(n, V), full[:, Q + K:]) < (1e-7 if dtype == "float32" else 8e-3)
    table, pages = pages_for_rows(dt, G, 2 * d, dv, pos, 4)
    q2 = torch.empty_like(q)
    ops.diff_split(dev(proj), dev(bias) if biased else None, rp, rot, H, G, d, dv, q2, None, None, table=table,
                   ring_pages=1 << 24, pages=pages)
    assert torch.equal(q2, q)
    for b, p in enumerate(pos):
        pk, pv = read_page(pages, table.cpu(), b, p, G, 2 * d, dv)
        assert torch.equal(pk, k[b]) and torch.equal(pv, v[b])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, dv", [(3, 6), (2, 64), (1, 200), (4, 256)])
def test_the_difference_of_the_maps_and_its_norm(dtype, H, dv):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(dv)
    dt = TORCH[dtype]
    maps = (torch.randn(5, 2 * H, dv, generator=g) + 0.5).to(dt)
    out = torch.empty(5, H, dv, dtype=dt, device="cuda")
    ops.diff_combine(dev(maps), 0.37, 1e-4, 0.7, out)
    m = maps.double().view(5, H, 2, dv)
    want = plain.rms(m[:, :, 0] - 0.37 * m[:, :, 1], 1e-4) * 0.7
    assert rel_err(out, want) < (1e-6 if dtype == "float32" else 8e-3)


# ---------------------------------------------------------------------------------------------
# the mixers' steps around the attention kernels, with keys that stand out
# ---------------------------------------------------------------------------------------------

class Sequence:
    """One sequence's cache for one mixer, driven as the engine drives it: steps of any size after one another,
    through `attend_and_commit`, pages of 64 in a ring when there is a window."""

    def __init__(self, dtype, nkv, dk, dv, window, seed=0, room=1100):
        from torchless_rs_amd.cache.cache import NO_RING
        from torchless_rs_amd.parts.base import Workspace
        self.dt, self.nkv, self.dk, self.dv = TORCH[dtype], nkv, dk, dv
        self.ring = -(-window // 64) if window else NO_RING
        n_seq = min(-(-room // 64), self.ring)
        n_pages = n_seq + 3
        order = torch.randperm(n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
        self.table = dev(torch.tensor([order[:n_seq]], dtype=torch.int32))
        shape = (n_pages, 2, nkv, 64, dk) if dk == dv else (n_pages, nkv * 64 * (dk + dv))
        self.pages = torch.full(shape, float("nan"), dtype=self.dt, device="cuda")
        self.ws = Workspace(torch.device("cuda"))
        self.length = 0

    def step(self, n_new):
        """(ctx, run) of a step that brings `n_new` rows after what the sequence holds."""
        from torchless_rs_amd.kernels import ops
        i32 = dict(dtype=torch.int32, device="cuda")
        cached = self.length
        offs, cols = ops.aligned_columns([cached], [n_new])
        ctx = types.SimpleNamespace(
            row_seq=torch.zeros(n_new, **i32), row_pos=torch.arange(cached, cached + n_new, **i32),
            cu_seqlens=torch.tensor([0, n_new], **i32), len_before=torch.tensor([cached], **i32),
            len_after=torch.tensor([cached + n_new], **i32), tile_off=torch.tensor(offs, **i32), all_single=n_new == 1,
            workspace=self.ws, n_rows=n_new, n_seqs=1, dtype=self.dt, max_new=n_new, tables={0: self.table},
            host={"n_new": np.asarray([n_new], dtype=np.int64), "len_before": np.asarray([cached], dtype=np.int64),
                  "aligned_cols": cols})
        group = types.SimpleNamespace(storage=[self.pages], ring_pages=self.ring)
        run = types.SimpleNamespace(kv_group=group, kv_layer=0, kv_group_index=0)
        self.length += n_new
        return ctx, run


def latent_steps(dtype, H, dk, dv, window, sinks, q, k, v, cuts, scale=1.0):
    """q, k, v [L, H, *] float: through `split_heads` and `attend_and_commit` in steps of `cuts` rows."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.attention_scored import attend_and_commit
    seq = Sequence(dtype, H, dk, dv, window)
    terms = ops.ScoreTerms(scale, window, None, dev(sinks.float()) if sinks is not None else None)
    outs, at = [], 0
    for n in cuts:
        ctx, run = seq.step(n)
        qf = dev(q[at:at + n].reshape(n, H * dk).float())
        kvf = dev(torch.cat([k[at:at + n].reshape(n, -1), v[at:at + n].reshape(n, -1)], dim=1).float())
        qs = torch.empty(n, H, dk, dtype=seq.dt, device="cuda")
        att = torch.empty(n, H, dv, dtype=seq.dt, device="cuda")
        if n == 1:
            ops.split_heads(qf, kvf, ctx.row_pos, H, H, dk, dv, qs, None, None, table=seq.table, ring_pages=seq.ring,
                            pages=seq.pages)
            ks = vs = None
        else:
            ks = torch.empty(n, H, dk, dtype=seq.dt, device="cuda")
            vs = torch.empty(n, H, dv, dtype=seq.dt, device="cuda")
            ops.split_heads(qf, kvf, ctx.row_pos, H, H, dk, dv, qs, ks, vs)
        attend_and_commit(ctx, run, qs, ks, vs, H, dk, dv, terms, None, att)
        outs.append(att.clone())
        at += n
    return torch.cat(outs)


def plain_heads(q, k, v, scale, window, sinks=None):
    """[L, H, dv] float64: softmax over the visible keys per head, with an optional sink."""
    s = (q.double().transpose(0, 1) @ k.double().transpose(0, 1).transpose(1, 2)) * scale
    a = plain.softmax_with_sink(s, plain.visible(q.shape[0], window), None if sinks is None else sinks.double())
    return (a @ v.double().transpose(0, 1)).transpose(0, 1)


ATT_TOL = {"float32": 2e-5, "bfloat16": 1.2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 2, 63, 64, 65, 100, 129])
@pytest.mark.parametrize("dk, dv", [(16, 16), (16, 8)])
def test_latent_heads_a_key_just_inside_and_just_outside_the_window(dtype, window, dk, dv):
    """One key far above all others: the row whose window still holds it puts nearly all weight on its
    value, the next row none; in prompts, in portions and decoded one by one, across page borders,
    with a sink that would otherwise take a fair share."""
    H = 2
    g = torch.Generator().manual_seed(window)
    for loud in (0, 5, 63, 64, 130):
        L = loud + window + 3
        q, k, v = torch.randn(L, H, dk, generator=g), torch.randn(L, H, dk, generator=g), torch.randn(L, H, dv, generator=g)
        k[loud] = 0
        k[loud, :, 0] = 30.0
        q[:, :, 0] = q[:, :, 0].abs() + 1.0
        v[loud] = 50.0
        dt = TORCH[dtype]
        q, k, v = q.to(dt).float(), k.to(dt).float(), v.to(dt).float()
        sinks = torch.tensor([1.0, -2.0])
        want = plain_heads(q, k, v, 1.0, window, sinks)
        edge = loud + window - 1
        tail = L - (loud + 1)
        for cuts in ([L], [loud + 1] + [1] * tail, [loud + 1, 2] + [tail - 2] if tail > 3 else [L]):
            got = latent_steps(dtype, H, dk, dv, window, sinks, q, k, v, cuts)
            assert rel_err(got, want) < ATT_TOL[dtype], (window, loud, cuts[:3])
            rows = got.float().mean(dim=(1, 2))
            assert rows[edge] > 25 and rows[edge + 1] < 25, (window, loud, cuts[:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_heads_a_far_key_the_first_tokens_and_the_sink_alone(dtype):
    H, dk, dv = 2, 32, 32
    g = torch.Generator().manual_seed(9)
    L = 700
    q, k, v = torch.randn(L, H, dk, generator=g), torch.randn(L, H, dk, generator=g), torch.randn(L, H, dv, generator=g)
    k[3] = 0
    k[3, :, 1] = 20.0
    q[-1, :, 1] = 3.0                     # the last query asks for position 3, far back
    v[3] = -40.0
    dt = TORCH[dtype]
    q, k, v = q.to(dt).float(), k.to(dt).float(), v.to(dt).float()
    want = plain_heads(q, k, v, 0.2, None, torch.zeros(H))
    for cuts in ([L], [650, 50], [699, 1], [1, 1, 1, 697]):
        got = latent_steps(dtype, H, dk, dv, None, torch.zeros(H), q, k, v, cuts, scale=0.2)
        assert rel_err(got, want) < ATT_TOL[dtype], cuts
        assert got[-1].float().mean() < -30
    # the first position sees itself and the sink: its weight is e^s / (e^s + e^sink), not 1
    s0 = (q[0] * k[0]).sum(-1).double() * 0.2
    share = torch.exp(s0) / (torch.exp(s0) + 1.0)
    assert rel_err(got[0], v[0].double() * share[:, None]) < ATT_TOL[dtype]
    # a sink far above every score takes all the weight
    got = latent_steps(dtype, H, dk, dv, None, torch.full((H,), 60.0), q[:40], k[:40], v[:40], [20, 20], scale=0.2)
    assert got.float().abs().max() < 1e-6


def diff_steps(dtype, H, G, d, dv, window, lam, post, eps, proj, cuts, scale=1.0, rot=None):
    """proj [L, 2Hd + 2Gd + G dv]: through `diff_split`, `attend_and_commit` and `diff_combine`."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.attention_scored import attend_and_commit
    seq = Sequence(dtype, G, 2 * d, dv, window)
    terms = ops.ScoreTerms(scale, window, None, None)
    outs, at = [], 0
    for n in cuts:
        ctx, run = seq.step(n)
        pr = dev(proj[at:at + n].float().contiguous())
        qs = torch.empty(n, 2 * H, 2 * d, dtype=seq.dt, device="cuda")
        maps = torch.empty(n, 2 * H, dv, dtype=seq.dt, device="cuda")
        if n == 1:
            ops.diff_split(pr, None, ctx.row_pos, rot, H, G, d, dv, qs, None, None, table=seq.table, ring_pages=seq.ring,
                           pages=seq.pages)
            ks = vs = None
        else:
            ks = torch.empty(n, G, 2 * d, dtype=seq.dt, device="cuda")
            vs = torch.empty(n, G, dv, dtype=seq.dt, device="cuda")
            ops.diff_split(pr, None, ctx.row_pos, rot, H, G, d, dv, qs, ks, vs)
        attend_and_commit(ctx, run, qs, ks, vs, G, 2 * d, dv, terms, None, maps)
        att = torch.empty(n, H, dv, dtype=seq.dt, device="cuda")
        ops.diff_combine(maps, lam, eps, post, att)
        outs.append(att.clone())
        at += n
    return torch.cat(outs)


def plain_diff(proj, H, G, d, dv, window, lam, post, eps, scale):
    L = proj.shape[0]
    Q, K = 2 * H * d, 2 * G * d
    q, k, v = proj[:, :Q].view(L, 2 * H, d), proj[:, Q:Q + K].view(L, 2 * G, d), proj[:, Q + K:].view(L, G, dv)
    out = torch.empty(L, H, dv, dtype=torch.float64)
    for h in range(H):
        gq = h // (H // G)
        a = [plain_heads(q[:, 2 * h + m:2 * h + m + 1], k[:, 2 * gq + m:2 * gq + m + 1], v[:, gq:gq + 1], scale, window)[:, 0]
             for m in range(2)]
        out[:, h] = plain.rms(a[0] - lam * a[1], eps) * post
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, d, dv", [(2, 1, 16, 32), (4, 2, 8, 24), (2, 2, 32, 64)])
def test_differential_maps_each_see_their_own_keys(dtype, H, G, d, dv):
    """A key that is loud in map 2 ONLY, far back among hundreds: the last query's map 2 puts its weight
    there while map 1 stays spread out, so the head's output is mean - lambda * loud value.  Keys of the
    wrong map, a lost map or a shared softmax would all show; so would a window that is one off."""
    g = torch.Generator().manual_seed(d)
    L = 400
    Q, K = 2 * H * d, 2 * G * d
    dt = TORCH[dtype]
    for window in (None, 130):
        loud = 7 if window is None else L - window           # far back, or the window's last key
        proj = torch.randn(L, Q + K + G * dv, generator=g) * 0.5
        k = proj[:, Q:Q + K].view(L, G, 2, d)
        k[loud, :, 1] = 0
        k[loud, :, 1, 2] = 25.0                              # map 2 of every KV head
        q = proj[:, :Q].view(L, H, 2, d)
        q[-1, :, 1, 2] = 2.0                                 # the last row's second map asks for it
        q[-1, :, 0, 2] = 2.0                                 # its first map would too, but map 1's key there is quiet
        v = proj[:, Q + K:].view(L, G, dv)
        v[loud] = 30.0
        proj = proj.to(dt).float()
        want = plain_diff(proj.double(), H, G, d, dv, window, 0.6, 0.7, 1e-5, 1.0)
        for cuts in ([L], [L - 1, 1], [loud + 1, L - loud - 3, 1, 1]):
            got = diff_steps(dtype, H, G, d, dv, window, 0.6, 0.7, 1e-5, proj, cuts)
            assert rel_err(got, want) < ATT_TOL[dtype] * 3, (window, cuts)
            # a1 - 0.6 * 30 dominates: after the norm every channel is close to -post
            assert got[-1].float().mean() < -0.6 and got[-2].float().mean() > -0.5
        if window is not None:                               # one row later the loud key has left the window
            more = torch.cat([proj, proj[-1:]])
            got = diff_steps(dtype, H, G, d, dv, window, 0.6, 0.7, 1e-5, more, [L, 1])
            assert rel_err(got, plain_diff(more.double(), H, G, d, dv, window, 0.6, 0.7, 1e-5, 1.0)) < ATT_TOL[dtype] * 3
            assert got[-1].float().mean() > -0.5


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def zoo(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("fanitar")
    out = {}
    for i, name in enumerate(NAMES):
        cfg = copy.deepcopy(CONFIGS[name])
        w = plain.random_weights(cfg, seed=40 + i)
        ps = some_prompts(cfg["vocab"], LENGTHS[name], seed=13 + i)
        out[name] = dict(dir=write_model(str(tmp / name), cfg, w), cfg=cfg, w=w, prompts=ps,
                         want=[plain.forward(w, cfg, p) for p in ps])
    return out


_engines = {}


def engine_for(zoo, name, dtype):
    from torchless_rs_amd.engine import Engine, load_model
    key = (name, dtype)
    if key not in _engines:
        _engines[key] = Engine(load_model(zoo[name]["dir"], dtype), max_tokens=64 * 20, max_slots=8)
    eng = _engines[key]
    assert not eng.cache.length, "a test left slots held"
    for g in eng.cache.groups:              # stale rows must never be read: make them NaN
        g.storage.fill_(float("nan"))
    return eng


def close(got, want, dtype, what):
    assert rel_err(got, want) < TOL[dtype], (what, rel_err(got, want))
    assert rms_err(got, want) < RMS[dtype], (what, rms_err(got, want))


def test_the_right_parts_and_caches_are_chosen(zoo):
    from torchless_rs_amd.parts.attention_diff import DifferentialAttentionMixer
    from torchless_rs_amd.parts.attention_latent import LatentAttentionMixer
    from torchless_rs_amd.parts.block import SandwichNormBlock
    from torchless_rs_amd.parts.norms import RMSNorm
    eng = engine_for(zoo, "mixed", "bfloat16")
    blocks = eng.model.blocks
    assert all(isinstance(b, SandwichNormBlock) for b in blocks)
    assert [type(b.mixer) for b in blocks] == [LatentAttentionMixer, DifferentialAttentionMixer] * 2
    assert blocks[2].ffn is None and blocks[0].ffn.activation == "swish_clamped"
    assert isinstance(eng.model.final_norm, RMSNorm)
    assert blocks[1].mixer.lam == pytest.approx(plain.diff_lambda({k: v.double() for k, v in zoo["mixed"]["w"].items()},
                                                                  "l1.mix.", 0.3), rel=1e-6)
    # eight runs, each with a place of its own in the cache: a layer that runs three times keeps three
    assert len(eng.runs) == 8
    places = {(r.kv_group_index, r.kv_layer) for r in eng.runs}
    assert len(places) == 8
    assert eng.runs[0].kv_group.ring_pages == 1 and eng.runs[1].kv_group.request.head_dim == 16


def test_which_attention_kernels_run(zoo, monkeypatch):
    """bfloat16 with head sizes the matrix cores take: the layers out of latents run the kernels with
    terms (their sink), the differential layers the kernels without, none the one that sums in float;
    a step of at most 16 rows applies the clamped gate in the product's epilogue, not in a kernel of its own."""
    from torchless_rs_amd.engine import SeqInput
    from torchless_rs_amd.kernels import ops
    eng, z = engine_for(zoo, "cores", "bfloat16"), zoo["cores"]
    calls = {"plain": 0, "terms": 0, "bare": 0, "act": 0}
    real_terms, real_bare = ops.attention_scored, ops.attention

    def no_plain(*a, **k):
        calls["plain"] += 1
        raise AssertionError("the float kernel ran")

    def terms(*a, **k):
        calls["terms"] += 1
        return real_terms(*a, **k)

    def bare(*a, **k):
        calls["bare"] += 1
        return real_bare(*a, **k)

    def act(*a, **k):
        calls["act"] += 1
        raise AssertionError("the gate ran in a kernel of its own")

    monkeypatch.setattr(ops, "attn_scored_plain", no_plain)
    monkeypatch.setattr(ops, "attention_scored", terms)
    monkeypatch.setattr(ops, "attention", bare)
    monkeypatch.setattr(ops, "act_mul", act)
    s = eng.alloc()
    eng.step([SeqInput(s, z["prompts"][2][:100], [99])])
    eng.step([SeqInput(s, z["prompts"][2][100:101], [0])])
    eng.free(s)
    # five runs a step (two passes over the first two layers, then the third): three out of latents, two differential
    assert calls == {"plain": 0, "terms": 6, "bare": 4, "act": 0}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_each_request_alone_and_whole(zoo, name, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    for p, want in zip(z["prompts"], z["want"]):
        s = eng.alloc()
        got = eng.step([SeqInput(s, p, list(range(len(p))))]).clone()
        eng.free(s)
        close(got, want, dtype, (name, len(p)))
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "cores"])
def test_the_stream_after_every_run_of_a_layer(zoo, name, dtype):
    from torchless_rs_amd.engine import Engine, SeqInput, load_model
    z = zoo[name]
    streams = []
    plain.forward(z["w"], z["cfg"], z["prompts"][2], streams)
    model = load_model(z["dir"], dtype)
    eng = Engine(model, max_tokens=256, use_graphs=False)
    seen = []
    for blk in model.blocks:
        inner = blk.forward

        def spy(ctx, run, x, *a, _inner=inner, **kw):
            _inner(ctx, run, x, *a, **kw)
            seen.append(x.clone())
        blk.forward = spy
    s = eng.alloc()
    eng.step([SeqInput(s, z["prompts"][2], [0])])
    eng.free(s)
    assert len(seen) == len(streams)
    for i, (got, want) in enumerate(zip(seen, streams)):
        assert got.dtype == torch.float32            # the residual sum is kept in 32 bits in both dtypes
        assert rel_err(got, want) < (2e-5 if dtype == "float32" else 4e-2), i
    eng.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prefill_against_decoding_token_by_token(zoo, name, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    for p, want in zip(z["prompts"][1:3], z["want"][1:3]):
        s = eng.alloc()
        rows = [eng.step([SeqInput(s, [t], [0])]).clone() for t in p]        # from the very first token
        eng.free(s)
        close(torch.cat(rows), want, dtype, (name, len(p), "token by token"))
    p, want = z["prompts"][3], z["want"][3]
    k = 40
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, p[:-k], list(range(len(p) - k)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in p[-k:]]
    eng.free(s)
    close(torch.cat(rows), want, dtype, (name, "prompt then 40 tokens"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("portion", [2, 3, 17, 64, 100])
def test_portions_of_a_prompt(zoo, name, dtype, portion):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    p, want = z["prompts"][3], z["want"][3]
    if portion < 4:
        p, want = p[:41], want[:41]
    s = eng.alloc()
    rows = []
    for at in range(0, len(p), portion):
        part = p[at:at + portion]
        rows.append(eng.step([SeqInput(s, part, list(range(len(part))))]).clone())
    eng.free(s)
    close(torch.cat(rows), want, dtype, (name, portion))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_against_each_alone_with_slots_and_pages_used_again(zoo, name, dtype):
    """All prompts in one step, then decoded together while the shorter ones end; a second batch takes
    the freed slots and pages (which hold the first batch's rows) and must give the same."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    tails = [0, 3, 9, 20]
    for turn in range(2):
        order = list(range(4)) if turn == 0 else [3, 1, 0, 2]
        slots = {i: eng.alloc() for i in order}
        heads = {i: len(z["prompts"][i]) - tails[i] for i in order}
        got = {i: [] for i in order}
        lg = eng.step([SeqInput(slots[i], z["prompts"][i][:heads[i]], list(range(heads[i]))) for i in order])
        at = 0
        for i in order:
            got[i].append(lg[at:at + heads[i]].clone())
            at += heads[i]
        live = [i for i in order if tails[i]]
        for i in order:
            if not tails[i]:
                eng.free(slots[i])
        step = 0
        while live:
            lg = eng.step([SeqInput(slots[i], [z["prompts"][i][heads[i] + step]], [0]) for i in live]).clone()
            for r, i in enumerate(live):
                got[i].append(lg[r:r + 1])
            step += 1
            for i in [i for i in live if step == tails[i]]:
                eng.free(slots[i])
            live = [i for i in live if step < tails[i]]
        for i in order:
            close(torch.cat(got[i]), z["want"][i], dtype, (name, turn, i))
        eng.cache.check()
    assert not eng.cache.length


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "ones", "cores", "heads"])
def test_long_decoding_past_windows_and_rings(zoo, name, dtype):
    """A short prompt, then 300 tokens one by one (through captured graphs): every window is passed
    and every ring wraps more than once, in every pass's own cache."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    ids = some_prompts(z["cfg"]["vocab"], [310], seed=78)[0]
    want = plain.forward(z["w"], z["cfg"], ids)
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, ids[:10], list(range(10)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[10:]]
    eng.free(s)
    close(torch.cat(rows), want, dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_batch_mates(zoo, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, "odd", dtype), zoo["odd"]
    p = z["prompts"][2]
    s = eng.alloc()
    alone = eng.step([SeqInput(s, p, [len(p) - 1])]).clone()
    eng.free(s)
    slots = [eng.alloc() for _ in range(3)]
    lg = eng.step([SeqInput(slots[0], z["prompts"][3], []), SeqInput(slots[1], p, [len(p) - 1]),
                   SeqInput(slots[2], z["prompts"][0], [0])]).clone()
    for s in slots:
        eng.free(s)
    assert rel_err(lg[0:1], alone) < (1e-6 if dtype == "float32" else 2e-2)


def test_greedy_generation_through_the_entry_point(zoo):
    from torchless_rs_amd import SamplingConfig, generate_until_eos
    for name in ("mixed", "ones"):
        eng, z = engine_for(zoo, name, "float32"), zoo[name]
        ps = z["prompts"][:3]
        out = generate_until_eos(eng, ps, SamplingConfig.greedy(), max_tokens=12)
        for p, r in zip(ps, out):
            assert r.tokens == plain.generate_greedy(z["w"], z["cfg"], p, 12), (name, len(p))
    # bfloat16 may turn a near-tie the other way: every token must be the plain argmax within the tolerance
    eng, z = engine_for(zoo, "cores", "bfloat16"), zoo["cores"]
    out = generate_until_eos(eng, z["prompts"][:2], SamplingConfig.greedy(), max_tokens=8)
    for p, r in zip(z["prompts"][:2], out):
        ids = list(p)
        assert len(r.tokens) == 8
        for t in r.tokens:
            lg = plain.forward(z["w"], z["cfg"], ids)[-1]
            assert float(lg.max() - lg[t]) <= 2 * TOL["bfloat16"] * float(lg.abs().max())
            ids.append(t)


def test_the_command_line_and_the_trace_replay(zoo, tmp_path):
    z = zoo["mixed"]
    p = z["prompts"][2]
    r = subprocess.run([sys.executable, os.path.join(REPO, "bin", "torchless"), "--temperature", "0", "--max-tokens", "6",
                        "--dtype", "float32", z["dir"], " ".join(map(str, p))], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    want = plain.generate_greedy(z["w"], z["cfg"], p, 6)
    assert " ".join(map(str, want)) in r.stdout, (r.stdout, want)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": p[:20], "want": [0, 19]}, {"id": "b", "tokens": p[:3], "want": [2]}], "end": ["b"]},
             {"step": 1, "entries": [{"id": "a", "tokens": [p[20]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [p[21]], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "logits"
    r = subprocess.run([sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", z["dir"], "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "23"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = z["cfg"]["vocab"]
    first = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    last = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists()
    want = z["want"][2]
    assert rel_err(first, torch.stack([want[0], want[19], want[2]])) < TOL["float32"]
    assert rel_err(last, want[21:22]) < TOL["float32"]


# ---------------------------------------------------------------------------------------------
# the new parts in a design of another arrangement
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_the_new_parts_serve_another_design(dtype):
    """A model that is none of the designs, from the registry's parts alone, with old and new blocks
    next to each other so that every kind of border between them is crossed: pre-norm around the older
    attention with rotation and SwiGLU; the block with norms on both sides around the older attention
    and SwiGLU, which do not know of it; pre-norm again; pre-norm around differential attention with a
    subset of its options (no biases, no rotation, a window) and the clamped gate; norms on both sides
    around attention out of latents without sink and gate and no feed-forward; the last two gone through
    twice with the vector of a pass before each (and no embedding added again)."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec, Run
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, I, nq, nkv, d, eps, window = 64, 70, 96, 4, 2, 16, 1e-5, 20
    rms = PartSpec("rmsnorm", {"size": H, "eps": eps})
    rot = PartSpec("rotary", {"head_dim": d, "theta": 100.0})
    swiglu = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I})
    consts = {"alpha": 1.2, "limit": 1.5, "shift": 0.5}

    def old_attention(position):
        return PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d, "window": window,
                                      "position": position})
    pre = PartSpec("pre_norm", {"mixer_norm_name": "n1.", "ffn_norm_name": "n2."})
    both = PartSpec("sandwich_norm", {"names": ("n1.", "n1b.", "n2.", "n2b.")})
    layers = [
        LayerSpec(prefix="h.0.", mixer=old_attention(rot), ffn=swiglu, mixer_norm=rms, ffn_norm=rms, block=pre),
        LayerSpec(prefix="h.1.", mixer=old_attention(PartSpec("none", {})), ffn=swiglu, mixer_norm=rms, ffn_norm=rms,
                  mixer_out_norm=rms, ffn_out_norm=rms, block=both),
        LayerSpec(prefix="h.2.", mixer=old_attention(rot), ffn=swiglu, mixer_norm=rms, ffn_norm=rms, block=pre),
        LayerSpec(prefix="h.3.", mixer=PartSpec("differential_attention", {
            "hidden_size": H, "n_heads": 2, "n_kv_heads": 1, "head_dim": d, "v_head_dim": 2 * d, "lambda_init": 0.35,
            "norm_eps": eps, "scale": 0.25, "window": 33}),
            ffn=PartSpec("gated", {"hidden_size": H, "intermediate_size": I, "activation": "swish_clamped",
                                   "activation_constants": consts}), mixer_norm=rms, ffn_norm=rms, block=pre),
        LayerSpec(prefix="h.4.", mixer=PartSpec("latent_attention", {
            "hidden_size": H, "n_heads": 2, "head_dim": d, "v_head_dim": 24, "q_rank": 20, "kv_rank": 12, "scale": 0.25,
            "norm_eps": eps}), ffn=None, mixer_norm=rms, ffn_norm=None, mixer_out_norm=rms, block=both),
    ]
    schedule = [Run(0), Run(1), Run(2), Run(3, entry=(0, 0)), Run(4), Run(3, entry=(0, 1)), Run(4)]
    spec = ModelSpec(hidden_size=H, vocab_size=V, embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H, "scale": 2.0}),
                     embedding_prefix="model.", layers=layers, schedule=schedule, final_norm=rms,
                     final_norm_prefix="model.norm.", head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}),
                     head_prefix="lm_head.",
                     stream_parts=[("passes.", PartSpec("pass_entry", {"hidden_size": H, "passes": 2, "name": "vec",
                                                                       "add_embedding": False}))])
    w = random_tensors(spec.weight_specs(), seed=6, std=0.2, norm_std=0.1, dtype=torch.bfloat16)
    W = {k: v.double().cpu() for k, v in w.items()}
    ids = some_prompts(V, [45], seed=9)[0]
    n = len(ids)
    pos = torch.arange(n)

    def lin(name, t):
        return t @ W[name].T

    def older(p, y, rotated):
        q, k, v = (lin(p + f"self_attn.{t}_proj.weight", y) for t in "qkv")
        q, k = q.view(n, nq, d), k.view(n, nkv, d)
        if rotated:
            q, k = plain.rotate(q, pos, 100.0, d), plain.rotate(k, pos, 100.0, d)
        k, v = k.repeat_interleave(nq // nkv, dim=1), v.view(n, nkv, d).repeat_interleave(nq // nkv, dim=1)
        return lin(p + "self_attn.o_proj.weight", plain_heads(q, k, v, d ** -0.5, window).reshape(n, nq * d))

    def silu_ffn(p, y):
        g, u = lin(p + "mlp.gate_proj.weight", y), lin(p + "mlp.up_proj.weight", y)
        return lin(p + "mlp.down_proj.weight", g / (1 + torch.exp(-g)) * u)

    def norm(name, t):
        return plain.rms(t, eps, W[name])

    x = W["model.embed_tokens.weight"][ids] * 2.0
    for p in ("h.0.", "h.1.", "h.2."):
        if p == "h.1.":
            x = x + norm(p + "n1b.weight", older(p, norm(p + "n1.weight", x), False))
            x = x + norm(p + "n2b.weight", silu_ffn(p, norm(p + "n2.weight", x)))
        else:
            x = x + older(p, norm(p + "n1.weight", x), True)
            x = x + silu_ffn(p, norm(p + "n2.weight", x))
    zero = {"h.3.mix.q.b": torch.zeros(4 * d, dtype=torch.float64), "h.3.mix.k.b": torch.zeros(2 * d, dtype=torch.float64),
            "h.3.mix.v.b": torch.zeros(2 * d, dtype=torch.float64), "h.4.mix.sink": torch.full((2,), -1e30, dtype=torch.float64),
            "h.4.mix.g": torch.zeros(48, H, dtype=torch.float64)}
    Wz = dict(W, **zero)
    for t in range(2):
        x = x + W["passes.vec"][t]
        y = norm("h.3.n1.weight", x)
        x = x + plain.differential_attention(y, Wz, "h.3.mix.", {"heads": 2, "kv_heads": 1, "dim": d, "vdim": 2 * d, "scale": 0.25,
                                                                  "diff": 0.35, "mask": {"size": 33}}, eps)
        y = norm("h.3.n2.weight", x)
        g = lin("h.3.mlp.gate_proj.weight", y).clamp(max=1.5)
        u = lin("h.3.mlp.up_proj.weight", y).clamp(-1.5, 1.5)
        x = x + lin("h.3.mlp.down_proj.weight", g * torch.sigmoid(1.2 * g) * (u + 0.5))
        y = norm("h.4.n1.weight", x)
        # (no sink: one far below every score; no gate: a zero projection gates by one half, undone here)
        a = plain.latent_attention(y, Wz, "h.4.mix.", {"heads": 2, "dim": d, "vdim": 24, "scale": 0.25}, eps) * 2.0
        x = x + norm("h.4.n1b.weight", a)
    want = lin("lm_head.weight", norm("model.norm.weight", x))
    model = Model(spec, None, TORCH[dtype], torch.device("cuda:0"))
    model.load_weights(TensorDict(w))
    eng = Engine(model, max_tokens=256)
    s = eng.alloc()
    got = [eng.step([SeqInput(s, ids[:30], list(range(30)))]).clone()]
    got += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[30:]]       # (steps of one row: norms cut in two at the borders)
    eng.free(s)
    close(torch.cat(got), want, dtype, "old and new blocks side by side")
    s = eng.alloc()
    got = [eng.step([SeqInput(s, ids[at:at + 7], list(range(len(ids[at:at + 7]))))]).clone() for at in range(0, n, 7)]
    eng.free(s)
    close(torch.cat(got), want, dtype, "the same in portions of seven")
    eng.close()
