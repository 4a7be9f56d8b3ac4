"""Sozetar on the GPU against the plain implementation of `plain_sozetar.py`: every
mechanism alone at the level of its kernel, then whole models of the tests' own sizes
through the engine: whole prompts, decoding token by token, portions down to two
tokens, unequal batches, slots and pages used again, long decoding past windows and
rings, the first tokens, and greedy generation through the entry point."""
import copy
import json
import os
import subprocess
import sys
import types

import numpy as np
import pytest
import torch

import plain_sozetar as plain
from test_sozetar_config import MIXED, att, layer
from util import rel_err, rms_err

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# largest difference as a share of the largest value (float32: the order of sums is all that differs);
# bfloat16 is held to the root mean square as well
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
RMS = {"float32": 1e-5, "bfloat16": 2.5e-2}

# a window that is no multiple of a page under a reader that looks back over three pages; heads of 40 and 24
WIDE = {"architecture": "Sozetar", "vocab": 200, "width": 96, "norm": {"eps": 1e-6}, "layers": [
    layer(att(6, 3, 40, 24, 0.16, window=70, temp=(0.3, 16)), ff=80),
    layer(att(6, 3, 40, 24, 0.16, window=130, temp=(0.2, 50), kv_from=0), ff=72),
]}
# what a model may happen to make 1 or equal: one head, as many KV heads as heads, a window of one (a
# position sees itself alone), of exactly one page and of two, a step of the factor on q at every position
ONES = {"architecture": "Sozetar", "vocab": 96, "width": 32, "norm": {"eps": 1e-4}, "layers": [
    layer(att(3, 3, 16, 16, 0.25, window=64, temp=(0.4, 1)), ff=32),
    layer(att(1, 1, 16, 16, 0.25, window=1)),
    layer(att(2, 2, 8, 8, 0.35, window=128), ff=8),
]}
# heads that the matrix cores take (64 and 32 wide, values of 64), grouped 4 to a KV head
CORES = {"architecture": "Sozetar", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "layers": [
    layer(att(8, 2, 64, 64, 0.125, window=100, temp=(0.3, 32)), ff=192),
    layer(att(8, 2, 64, 64, 0.125, window=100, kv_from=0), ff=192),
    layer(att(4, 1, 32, 64, 0.18, temp=(0.3, 40)), ff=64),
    layer(att(4, 1, 32, 64, 0.18, window=40, kv_from=2)),
]}
# sizes that no kernel's fast way takes: a width that is no multiple of 8, heads of 12 and 20, 5 heads, an odd vocabulary
ODD = {"architecture": "Sozetar", "vocab": 131, "width": 100, "norm": {"eps": 1e-5}, "layers": [
    layer(att(5, 5, 12, 20, 0.29, window=33, temp=(0.25, 10)), ff=50),
    layer(att(5, 5, 12, 20, 0.29, kv_from=0, temp=(0.6, 2.5)), ff=36),
]}
CONFIGS = {"mixed": MIXED, "wide": WIDE, "ones": ONES, "cores": CORES, "odd": ODD}
LENGTHS = {"mixed": [1, 7, 23, 70], "wide": [3, 66, 150, 290], "ones": [2, 65, 130, 200], "cores": [5, 64, 129, 330],
           "odd": [4, 33, 67, 140]}
NAMES = list(CONFIGS)


# ---------------------------------------------------------------------------------------------
# the kernels one by one
# ---------------------------------------------------------------------------------------------

def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype is not None else t.to("cuda")


@pytest.mark.parametrize("H", [32, 100, 1024, 1030, 4096])
@pytest.mark.parametrize("out_dtype", DTYPES)
def test_layer_norm_alone_with_bias_and_into_the_stream(H, out_dtype):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(H)
    z = torch.randn(5, H, generator=g) * 3 + 1.5
    w, b, x = 1 + 0.3 * torch.randn(H, generator=g), torch.randn(H, generator=g), torch.randn(5, H, generator=g)
    odt = TORCH[out_dtype]
    tol = 1e-5 if out_dtype == "float32" else 8e-3
    out = torch.empty(5, H, dtype=odt, device="cuda")
    ops.layernorm(dev(z), dev(w), 1e-5, out)
    assert rel_err(out, plain.layer_norm(z.double(), w.double(), 1e-5)) < tol
    ops.layernorm(dev(z), dev(w), 1e-5, out, bias=dev(b))
    assert rel_err(out, plain.layer_norm((z + b).double(), w.double(), 1e-5)) < tol
    xs = dev(x.clone())
    ops.layernorm(dev(z), dev(w), 1e-5, out, add_to=xs, bias=dev(b))
    want = x.double() + plain.layer_norm((z + b).double(), w.double(), 1e-5)
    assert rel_err(xs, want) < 1e-5 and rel_err(out, want) < tol         # the stream itself stays float32
    xs = dev(x.clone())
    ops.layernorm(dev(z), dev(w), 1e-5, None, add_to=xs)
    assert rel_err(xs, x.double() + plain.layer_norm(z.double(), w.double(), 1e-5)) < 1e-5


def test_a_row_far_from_zero_keeps_its_variance():
    """mean >> deviation: a variance taken as mean of squares minus square of mean would lose it."""
    from torchless_rs_amd.kernels import ops
    z = 1000.0 + torch.randn(3, 64, generator=torch.Generator().manual_seed(0)) * 0.01
    out = torch.empty(3, 64, device="cuda")
    ops.layernorm(dev(z), torch.ones(64, device="cuda"), 1e-12, out)
    assert rel_err(out, plain.layer_norm(z.double(), torch.ones(64, dtype=torch.float64), 1e-12)) < 2e-3


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_gate_functions(activation):
    from torchless_rs_amd.kernels import ops
    gu = torch.randn(4, 2 * 50, generator=torch.Generator().manual_seed(1)) * 3
    out = torch.empty(4, 50, device="cuda")
    ops.act_mul(dev(gu), out, activation)
    g, u = gu[:, :50].double(), gu[:, 50:].double()
    want = (plain.gelu_tanh(g) if activation == "gelu_tanh" else g / (1 + torch.exp(-g))) * u
    assert rel_err(out, want) < 1e-6


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("K", [128, 192])                  # the ring of LDS stages takes multiples of 128, the other kernel the rest
@pytest.mark.parametrize("M", [1, 8, 16, 17, 64, 100, 128, 300])
def test_the_gate_function_in_the_epilogue_of_the_product(activation, K, M):
    """gate and up rows interleaved in blocks of 32: every kernel that a row count selects applies
    act(gate) * up to its float sums itself; above the kernels' own rows the library's product is
    followed by the same function on bfloat16 pairs."""
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.linear import interleave_pairs
    g = torch.Generator().manual_seed(M + K)
    I = 96
    a = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
    wg, wu = ((torch.randn(I, K, generator=g) * 0.2).to(torch.bfloat16) for _ in range(2))
    w = dev(interleave_pairs(wg, wu))
    out = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    if M > ops.own_rows(K):
        gu = torch.empty(M, 2 * I, dtype=torch.bfloat16, device="cuda")
        ops.gemm_library(dev(a), w, gu)
        ops.silu_mul_pairs(gu, out, activation)
    elif M > 16:
        ops.gemm_mid_bf16(dev(a), w, out, 1, silu_pair=True, pair_act=activation)
    else:
        ops.gemm_bf16(dev(a), w, out, silu_pair=True, pair_act=activation)
    gate, up = a.double() @ wg.double().T, a.double() @ wu.double().T
    act = plain.gelu_tanh(gate) if activation == "gelu_tanh" else gate / (1 + torch.exp(-gate))
    assert rel_err(out, act * up) < (2e-2 if M > ops.own_rows(K) else 6e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, nkv, dk, dv, ng, temp, normed, biased", [
    (4, 2, 16, 32, 4, (0.5, 3), True, True),
    (6, 3, 40, 24, 6, (0.3, 16), True, False),
    (2, 0, 24, 8, 2, None, True, True),            # a mixer that reads another's keys: q and the gate alone
    (3, 3, 8, 8, 0, (0.4, 1), False, True),        # no norm, no gate
])
def test_the_split_of_the_projection(dtype, nq, nkv, dk, dv, ng, temp, normed, biased):
    from torchless_rs_amd.kernels import ops
    g = torch.Generator().manual_seed(nq * 100 + dk)
    Q, K, V = nq * dk, nkv * dk, nkv * dv
    n = 9
    proj = torch.randn(n, Q + K + V + ng, generator=g) * 2
    pos = torch.tensor([0, 1, 2, 3, 5, 15, 16, 47, 1000], dtype=torch.int32)
    bias = torch.randn(Q + K + V + ng, generator=g) if biased else None
    if bias is not None and ng:
        bias[Q + K + V:] = 0
    wq, wk = 1 + 0.3 * torch.randn(Q, generator=g), 1 + 0.3 * torch.randn(max(K, 1), generator=g)[:K]
    terms = ops.ProjectionTerms(bias=dev(bias) if biased else None, q_norm=dev(wq) if normed else None,
                                k_norm=dev(wk) if normed and nkv else None, eps=1e-5, temperature=temp)
    dt = TORCH[dtype]
    q = torch.empty(n, nq, dk, dtype=dt, device="cuda")
    k = torch.empty(n, max(nkv, 1), dk, dtype=dt, device="cuda")[:, :nkv].contiguous()
    v = torch.empty(n, max(nkv, 1), dv, dtype=dt, device="cuda")[:, :nkv].contiguous()
    gate = torch.empty(n, ng, device="cuda") if ng else None
    ops.split_projection(dev(proj), dev(pos), terms, nq, nkv, dk, dv, ng, q, k if nkv else None, v if nkv else None, gate)
    full = proj.double() + (bias.double() if biased else 0)
    wq_, wk_ = (wq.double(), wk.double()) if normed else (None, None)
    want_q = plain.rms_over_projection(full[:, :Q], wq_, 1e-5) if normed else full[:, :Q]
    if temp:
        t = 1 + temp[0] * torch.log(torch.floor((pos.double() + 1) / temp[1]) + 1)
        want_q = want_q * t[:, None]
    tol = 1e-5 if dtype == "float32" else 8e-3
    assert rel_err(q.view(n, Q), want_q) < tol
    if nkv:
        want_k = plain.rms_over_projection(full[:, Q:Q + K], wk_, 1e-5) if normed else full[:, Q:Q + K]
        assert rel_err(k.view(n, K), want_k) < tol
        assert rel_err(v.view(n, V), full[:, Q + K:Q + K + V]) < tol
    if ng:
        assert rel_err(gate, torch.sigmoid(full[:, Q + K + V:])) < 1e-6


def attention_case(dtype, nq, nkv, dk, dv, cached, new, window, slopes, sinks, gated, seed, craft=None,
                   scale=0.3):
    """Sequences with `cached[b]` positions in pages (in a ring with a window) and `new[b]` rows in the
    step; returns (got, want) for the step's rows.  `craft(b, q, k, v)` may change a sequence's
    tensors (q [L, nq, dk] over all positions, of which the last new[b] are asked)."""
    from torchless_rs_amd.cache.cache import NO_RING
    from torchless_rs_amd.kernels import ops
    from torchless_rs_amd.parts.base import Workspace
    g = torch.Generator().manual_seed(seed)
    dt = TORCH[dtype]
    B = len(cached)
    ring = -(-window // 64) if window else NO_RING
    seqs = []
    for b in range(B):
        L = cached[b] + new[b]
        q, k, v = (torch.randn(L, nq, dk, generator=g), torch.randn(L, nkv, dk, generator=g),
                   torch.randn(L, nkv, dv, generator=g))
        if craft:
            craft(b, q, k, v)
        seqs.append([t.to(dt) for t in (q, k, v)])        # what both sides see is what the dtype holds
    pages_of = [min(-(-(cached[b] + new[b]) // 64), ring) for b in range(B)]
    n_pages = sum(pages_of) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    stride = max(pages_of)
    table = torch.zeros(B, stride, dtype=torch.int32)
    for b in range(B):
        for i in range(pages_of[b]):
            table[b, i] = order.pop()
    # (the shape of the cache's storage: values as wide as keys lie as [K|V, kv head, 64, d])
    shape = (n_pages, 2, nkv, 64, dk) if dk == dv else (n_pages, nkv * 64 * (dk + dv))
    pages = torch.full(shape, float("nan"), dtype=dt, device="cuda")
    table = dev(table)
    i32 = dict(dtype=torch.int32, device="cuda")
    # the cached positions go into the pages as a step of their own would have put them
    if sum(cached):
        ck = torch.cat([seqs[b][1][:cached[b]] for b in range(B)])
        cv = torch.cat([seqs[b][2][:cached[b]] for b in range(B)])
        rs = torch.tensor([b for b in range(B) for _ in range(cached[b])], **i32)
        rp = torch.tensor([p for b in range(B) for p in range(cached[b])], **i32)
        ops.kv_commit_wide(dev(ck), dev(cv), rs, rp, torch.tensor(cached, **i32), table, ring, pages)
    rows = [(b, cached[b] + i) for b in range(B) for i in range(new[b])]
    n = len(rows)
    q = dev(torch.cat([seqs[b][0][cached[b]:] for b in range(B)]))
    k_new = dev(torch.cat([seqs[b][1][cached[b]:] for b in range(B)]))
    v_new = dev(torch.cat([seqs[b][2][cached[b]:] for b in range(B)]))
    cu = np.concatenate([[0], np.cumsum(new)])
    all_single = all(x == 1 for x in new)
    len_after = torch.tensor([c + x for c, x in zip(cached, new)], **i32)
    offs, cols = ops.aligned_columns(cached, new)
    ctx = types.SimpleNamespace(
        row_seq=torch.tensor([r[0] for r in rows], **i32), row_pos=torch.tensor([r[1] for r in rows], **i32),
        cu_seqlens=torch.tensor(cu, **i32), len_before=torch.tensor(cached, **i32), len_after=len_after,
        tile_off=torch.tensor(offs, **i32),
        all_single=all_single, workspace=Workspace(torch.device("cuda")), n_rows=n, n_seqs=B, dtype=dt,
        max_new=max(new), host={"n_new": np.asarray(new, dtype=np.int64), "len_before": np.asarray(cached, dtype=np.int64),
                                "aligned_cols": cols})
    gate = torch.rand(n, nq, generator=g) if gated else None
    terms = ops.ScoreTerms(scale, window, dev(slopes.float()) if slopes is not None else None,
                           dev(sinks.float()) if sinks is not None else None)
    out = torch.empty(n, nq, dv, dtype=dt, device="cuda")
    if all_single:      # one token a sequence: the step's keys go into the pages first
        ops.kv_commit_wide(k_new, v_new, ctx.row_seq, ctx.row_pos, len_after, table, ring, pages)
        ops.attention_scored(q, None, None, pages, nkv, dv, table, ring, ctx, len_after, terms,
                             dev(gate) if gated else None, out)
    else:
        vt = None
        if ops.scored_on_matrix_cores(dt, dk, dv):        # the matrix cores read the step's values along the keys
            vt = torch.full((nkv, dv, cols), float("nan"), dtype=dt, device="cuda")
            ops.v_tiles_rows(v_new, vt, ctx.cu_seqlens, ctx.tile_off, ctx.len_before, len_after)
        ops.attention_scored(q, k_new, v_new, pages, nkv, dv, table, ring, ctx, ctx.len_before, terms,
                             dev(gate) if gated else None, out, vt_new=vt)
    want = torch.cat([plain.attend(seqs[b][0].double(), seqs[b][1].double(), seqs[b][2].double(), scale,
                                   slopes, sinks, window, first_row=cached[b])[cached[b]:] for b in range(B)])
    if gated:
        want = want * gate.double()[:, :, None]
    return out, want


ATT_TOL = {"float32": 2e-5, "bfloat16": 1.2e-2}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("what", ["nothing", "slopes", "sink", "window", "gate", "all"])
@pytest.mark.parametrize("nq, nkv, dk, dv", [(4, 2, 16, 32), (6, 3, 40, 24), (8, 2, 64, 64), (4, 1, 32, 64), (1, 1, 8, 8),
                                             (6, 1, 48, 48), (20, 1, 128, 128), (3, 3, 80, 80), (2, 1, 256, 256),
                                             (34, 2, 96, 96)])
def test_attention_terms_one_by_one(dtype, what, nq, nkv, dk, dv):
    slopes = plain.head_slopes(nq) if what in ("slopes", "all") else None
    sinks = torch.linspace(-1, 2, nq, dtype=torch.float64) if what in ("sink", "all") else None
    window = 37 if what in ("window", "all") else None
    gated = what in ("gate", "all")
    # prompts, prompts that go on from cached positions, and single tokens, in one call each
    for cached, new in (([0, 0], [70, 9]), ([64, 3, 130], [5, 66, 2]), ([5, 64, 199], [1, 1, 1])):
        got, want = attention_case(dtype, nq, nkv, dk, dv, cached, new, window, slopes, sinks, gated, seed=len(what))
        assert rel_err(got, want) < ATT_TOL[dtype], (what, cached, new)


def test_the_matrix_cores_serve_the_shapes_they_take(monkeypatch):
    """bfloat16 with values as wide as keys and head sizes in steps of 16 never reaches the plain kernel,
    in prompts, in portions after cached positions and in single-token steps; other shapes always do."""
    from torchless_rs_amd.kernels import ops
    calls = []
    plain_kernel = ops.attn_scored_plain
    monkeypatch.setattr(ops, "attn_scored_plain", lambda *a, **k: (calls.append(1), plain_kernel(*a, **k)))
    sinks = torch.zeros(4, dtype=torch.float64)
    for cached, new in (([0, 0], [70, 9]), ([64, 3], [5, 66]), ([5, 64, 199], [1, 1, 1])):
        for dk in (16, 48, 128):
            attention_case("bfloat16", 4, 2, dk, dk, cached, new, 37, plain.head_slopes(4), sinks, True, seed=1)
        assert not calls
    attention_case("bfloat16", 4, 2, 16, 32, [3], [5], None, None, sinks, False, seed=1)
    attention_case("bfloat16", 4, 2, 24, 24, [3], [1], None, None, sinks, False, seed=1)
    attention_case("float32", 4, 2, 16, 16, [3], [5], None, None, sinks, False, seed=1)
    assert len(calls) == 3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 2, 63, 64, 65, 72, 128, 129])
@pytest.mark.parametrize("single", [False, True])
def test_a_key_that_stands_out_just_inside_and_just_outside_the_window(dtype, window, single):
    """One key gets a score far above all others: the row whose window still holds it puts nearly
    all weight on its value, the next row none.  Misplacing the window's edge by one shows as a
    wholly different output, in prompts and in single-token steps, across page borders."""
    nq, nkv, dk, dv = 4, 2, 16, 16
    for loud in (0, 3, 63, 64, 100):           # position of the loud key
        L = loud + window + 2

        def craft(b, q, k, v):
            k[loud] = 0
            k[loud, :, 0] = 30.0
            q[:, :, 0] = q[:, :, 0].abs() + 1.0       # every query likes it
            v[loud] = 50.0

        edge = loud + window - 1                     # the last position that sees it
        if single:
            for p in (edge, edge + 1):
                got, want = attention_case(dtype, nq, nkv, dk, dv, [p], [1], window, None,
                                           torch.zeros(nq, dtype=torch.float64), False, 5, craft, scale=1.0)
                assert rel_err(got, want) < ATT_TOL[dtype], (window, loud, p)
                assert (got.float().mean() > 25) == (p == edge)
        else:
            for cached in (0, min(loud + 1, L - 2), 64 if L > 66 else 1):
                got, want = attention_case(dtype, nq, nkv, dk, dv, [cached], [L - cached], window, None,
                                           torch.zeros(nq, dtype=torch.float64), False, 5, craft, scale=1.0)
                assert rel_err(got, want) < ATT_TOL[dtype], (window, loud, cached)
                rows = got.float().mean(dim=(1, 2))
                if edge >= cached:
                    assert rows[edge - cached] > 25
                assert rows[edge + 1 - cached] < 25


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_among_hundreds_and_the_sink_alone(dtype):
    nq, nkv, dk, dv = 4, 1, 32, 64

    def craft(b, q, k, v):
        k[7] = 0
        k[7, :, 1] = 20.0
        q[-1, :, 1] = 3.0                # the last query asks for position 7
        v[7] = -40.0

    for cached, new in (([0], [700]), ([650], [50]), ([699], [1])):
        got, want = attention_case(dtype, nq, nkv, dk, dv, cached, new, None, plain.head_slopes(nq) * 0.01,
                                   torch.zeros(nq, dtype=torch.float64), False, 11, craft, scale=1.0)
        assert rel_err(got, want) < ATT_TOL[dtype]
        assert got[-1].float().mean() < -30
    # a sink far above every score takes all the weight: the output goes to zero, not to an average
    got, want = attention_case(dtype, nq, nkv, dk, dv, [10], [20], None, None, torch.full((nq,), 40.0, dtype=torch.float64),
                               False, 12)
    assert got.float().abs().max() < 1e-6 and want.abs().max() < 1e-6


@pytest.mark.parametrize("window", [None, 1000])
@pytest.mark.parametrize("nq, nkv, d", [(8, 2, 64), (4, 1, 128), (6, 3, 48), (2, 2, 256)])
def test_single_tokens_over_long_contexts_in_several_splits(nq, nkv, d, window):
    """Sequences of very unequal lengths, one token each: the keys of the long ones are cut over several
    workgroups whose sums are merged; the sink must count once, in whichever split, and the gate once."""
    sinks = torch.linspace(-2, 3, nq, dtype=torch.float64)
    for cached in ([2500, 70, 1300], [4000], [63, 64, 65, 1]):
        got, want = attention_case("bfloat16", nq, nkv, d, d, cached, [1] * len(cached), window,
                                   plain.head_slopes(nq) * 0.05, sinks, True, seed=d)
        assert rel_err(got, want) < ATT_TOL["bfloat16"], (cached,)


# ---------------------------------------------------------------------------------------------
# whole models through the engine
# ---------------------------------------------------------------------------------------------

def write_model(folder, cfg, weights):
    """config.json and model.safetensors, written with the test's own few lines."""
    import struct
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, t in weights.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes() if t.dtype != torch.bfloat16 \
            else t.contiguous().view(torch.int16).numpy().tobytes()
        header[name] = {"dtype": {torch.bfloat16: "BF16", torch.float32: "F32"}[t.dtype], "shape": list(t.shape),
                        "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(header).encode()
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"".join(blobs))
    return folder


def some_prompts(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


@pytest.fixture(scope="module")
def zoo(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("sozetar")
    out = {}
    for i, name in enumerate(NAMES):
        cfg = copy.deepcopy(CONFIGS[name])
        w = plain.random_weights(cfg, seed=20 + i)
        ps = some_prompts(cfg["vocab"], LENGTHS[name], seed=3 + i)
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


def test_the_right_parts_and_kernels_are_chosen(zoo):
    from torchless_rs_amd.parts.attention_scored import ScoredAttentionMixer
    from torchless_rs_amd.parts.block import OutputNormBlock
    from torchless_rs_amd.parts.norms import LayerNorm
    eng = engine_for(zoo, "mixed", "bfloat16")
    blocks = eng.model.blocks
    assert all(isinstance(b, OutputNormBlock) and isinstance(b.mixer, ScoredAttentionMixer) for b in blocks)
    assert blocks[1].ffn is None and blocks[0].ffn.activation == "gelu_tanh"
    assert isinstance(eng.model.final_norm, LayerNorm) and not blocks[1].mixer.own_kv
    assert blocks[0].mixer.slopes.tolist() == pytest.approx(plain.head_slopes(4).tolist())
    assert eng.runs[0].kv_group.ring_pages == 1 and eng.runs[2].kv_group.request.v_head_dim == 8


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
def test_the_stream_after_every_layer(zoo, dtype):
    """Layer by layer: the engine's residual stream, read after each block through a model cut
    short, against the plain implementation's."""
    from torchless_rs_amd.engine import Engine, SeqInput, load_model
    z = zoo["mixed"]
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
@pytest.mark.parametrize("name", ["mixed", "ones", "cores"])
def test_long_decoding_past_windows_and_rings(zoo, name, dtype):
    """A short prompt, then 300 tokens one by one (through captured graphs): every window is passed,
    every ring wraps more than once, the factor on q steps up many times."""
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, name, dtype), zoo[name]
    ids = some_prompts(z["cfg"]["vocab"], [310], seed=77)[0]
    want = plain.forward(z["w"], z["cfg"], ids)
    s = eng.alloc()
    rows = [eng.step([SeqInput(s, ids[:10], list(range(10)))]).clone()]
    rows += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[10:]]
    eng.free(s)
    close(torch.cat(rows), want, dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_batch_mates(zoo, dtype):
    from torchless_rs_amd.engine import SeqInput
    eng, z = engine_for(zoo, "wide", dtype), zoo["wide"]
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
# the new parts in designs of other arrangements
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_the_new_parts_serve_other_designs(dtype):
    """Two models that are neither design, from the registry's parts alone.  One: the output-norm block
    around the older parts (attention without terms, SwiGLU, RMSNorm), which do not know of it.  Two: the
    pre-norm block around the attention with a subset of its terms (a sink and a window: no biases, no
    norm of q and k, no slopes, no gate, no factor on q), layer norm before the sublayers and a gelu gate."""
    from torchless_rs_amd.engine import Engine, SeqInput
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.parts import LayerSpec, ModelSpec, PartSpec, Run
    from torchless_rs_amd.weights import TensorDict, random_tensors
    H, V, I, nq, nkv, d, L, eps, window = 64, 70, 96, 4, 2, 16, 2, 1e-5, 20
    rms = PartSpec("rmsnorm", {"size": H, "eps": eps})
    ln = PartSpec("layernorm", {"size": H, "eps": eps})
    older = [LayerSpec(prefix=f"h.{i}.",
                       mixer=PartSpec("attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                    "window": window, "position": PartSpec("none", {})}),
                       ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
                       mixer_norm=rms, ffn_norm=rms,
                       block=PartSpec("output_norm", {"mixer_norm_name": "n1.", "ffn_norm_name": "n2."})) for i in range(L)]
    subset = [LayerSpec(prefix=f"h.{i}.",
                        mixer=PartSpec("scored_attention", {"hidden_size": H, "n_heads": nq, "n_kv_heads": nkv, "head_dim": d,
                                                            "window": window, "sink": True, "prefix": "self_attn."}),
                        ffn=PartSpec("gated", {"hidden_size": H, "intermediate_size": I, "activation": "gelu_tanh"}),
                        mixer_norm=ln, ffn_norm=ln,
                        block=PartSpec("pre_norm", {"mixer_norm_name": "n1.", "ffn_norm_name": "n2."})) for i in range(L)]
    ids = some_prompts(V, [45], seed=8)[0]

    def lin(w, name, t):
        return t @ w[name].double().T

    for layers, final in ((older, rms), (subset, ln)):
        spec = ModelSpec(hidden_size=H, vocab_size=V, embedding=PartSpec("tokens", {"vocab_size": V, "hidden_size": H}),
                         embedding_prefix="model.", layers=layers, schedule=[Run(i) for i in range(L)],
                         final_norm=final, final_norm_prefix="model.norm.",
                         head=PartSpec("linear", {"vocab_size": V, "hidden_size": H}), head_prefix="lm_head.")
        w = random_tensors(spec.weight_specs(), seed=4, std=0.2, norm_std=0.1, dtype=torch.bfloat16)
        model = Model(spec, None, TORCH[dtype], torch.device("cuda:0"))
        model.load_weights(TensorDict(w))
        eng = Engine(model, max_tokens=256)
        x = w["model.embed_tokens.weight"].double()[ids]
        n = len(ids)
        for i in range(L):
            p = f"h.{i}."
            if layers is older:
                q, k, v = (lin(w, p + f"self_attn.{t}_proj.weight", x) for t in "qkv")
                a = plain.attend(q.view(n, nq, d), k.view(n, nkv, d), v.view(n, nkv, d), d ** -0.5, None, None, window)
                x = x + plain.rms_over_projection(lin(w, p + "self_attn.o_proj.weight", a.reshape(n, nq * d)),
                                                  w[p + "n1.weight"].double(), eps)
                g, u = lin(w, p + "mlp.gate_proj.weight", x), lin(w, p + "mlp.up_proj.weight", x)
                x = x + plain.rms_over_projection(lin(w, p + "mlp.down_proj.weight", g / (1 + torch.exp(-g)) * u),
                                                  w[p + "n2.weight"].double(), eps)
            else:
                y = plain.layer_norm(x, w[p + "n1.weight"].double(), eps)
                q, k, v = (lin(w, p + f"self_attn.{t}", y) for t in "qkv")
                a = plain.attend(q.view(n, nq, d), k.view(n, nkv, d), v.view(n, nkv, d), d ** -0.5, None,
                                 w[p + "self_attn.sink"].double(), window)
                x = x + lin(w, p + "self_attn.o", a.reshape(n, nq * d))
                y = plain.layer_norm(x, w[p + "n2.weight"].double(), eps)
                x = x + lin(w, p + "mlp.down_proj.weight",
                            plain.gelu_tanh(lin(w, p + "mlp.gate_proj.weight", y)) * lin(w, p + "mlp.up_proj.weight", y))
        nf = w["model.norm.weight"].double()
        want = lin(w, "lm_head.weight", plain.rms_over_projection(x, nf, eps) if layers is older else plain.layer_norm(x, nf, eps))
        s = eng.alloc()
        got = [eng.step([SeqInput(s, ids[:30], list(range(30)))]).clone()]
        got += [eng.step([SeqInput(s, [t], [0])]).clone() for t in ids[30:]]
        eng.free(s)
        close(torch.cat(got), want, dtype, "older parts in the new block" if layers is older else "a subset of the terms")
        eng.close()
