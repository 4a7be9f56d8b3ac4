"""Fanitar without a GPU: the configuration's reader, the model as a list of parts, the order
of runs with its passes, the tensor names, and the plain implementation's own mechanisms."""
import copy
import math

import pytest
import torch

import plain_fanitar as plain
from torchless_rs_amd.config import ConfigError, FanitarConfig
from torchless_rs_amd.config.base import config_from_dict
from torchless_rs_amd.models import model_spec_for


def latent(heads, dim, vdim, q_rank, kv_rank, scale, window=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    return m


def diff(heads, kv_heads, dim, vdim, scale, lam, rot=None, window=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": lam}
    if rot:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if window:
        m["mask"] = {"size": window}
    return m


def layer(mixer, ff=None, limit=None):
    kind = "latent_attention" if "q_rank" in mixer else "attention"
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


# both mixers, a layer without a feed-forward, three passes over the two layers in the middle
MIXED = {"architecture": "Fanitar", "vocab": 160, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
         "logit_scale": 0.5, "loop": {"start": 1, "stop": 3, "times": 3}, "layers": [
             layer(latent(2, 16, 8, 24, 40, 0.25, window=20), ff=96, limit=0.7),
             layer(diff(4, 2, 8, 24, 0.35, 0.3, rot=(1000.0, 4)), ff=80, limit=2.5),
             layer(latent(4, 8, 8, 16, 16, 0.3)),
             layer(diff(2, 2, 16, 32, 0.25, 0.8, rot=(50.0, 16)), ff=48, limit=1.5),
         ]}


def test_every_key_is_read_and_written_back():
    cfg = config_from_dict(copy.deepcopy(MIXED))
    assert isinstance(cfg, FanitarConfig)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.embedding_scale, cfg.logit_scale) == (160, 64, 3.0, 0.5)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 3)
    a, b, c, d = cfg.layers
    assert (a.mixer.q_rank, a.mixer.kv_rank, a.mixer.window, a.limit) == (24, 40, 20, 0.7)
    assert (b.mixer.kv_heads, b.mixer.rot_dims, b.mixer.rot_base, b.mixer.diff) == (2, 4, 1000.0, 0.3)
    assert c.ff is None and c.mixer.window is None and d.mixer.rot_dims == 16
    again = config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()
    for l, e in zip(cfg.to_dict()["layers"], MIXED["layers"]):
        assert l["mixer"] == e["mixer"] and l["mlp"] == e["mlp"]


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "no mixer of type"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "not a multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), "rotated channels"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 3), "rotated channels"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("dim", 200), "not served"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("dim", 300), "not served"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop over layers"),
    (lambda c: c["loop"].__setitem__("stop", 1), "loop over layers"),
    (lambda c: c["loop"].__setitem__("times", 0), "times"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_what_cannot_be_served_is_refused(change, text):
    cfg = copy.deepcopy(MIXED)
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


def test_the_model_as_parts_and_the_order_of_runs():
    spec = model_spec_for(config_from_dict(copy.deepcopy(MIXED)))
    assert [(r.layer, r.entry) for r in spec.schedule] == [
        (0, None), (1, (0, 0)), (2, None), (1, (0, 1)), (2, None), (1, (0, 2)), (2, None), (3, None)]
    assert [(r.layer, None if r.entry is None else r.entry[1]) for r in spec.schedule] == \
        [(i, t) for i, t in plain.order_of_runs(MIXED)]
    kinds = [l.mixer.kind for l in spec.layers]
    assert kinds == ["latent_attention", "differential_attention", "latent_attention", "differential_attention"]
    assert all(l.block.kind == "sandwich_norm" for l in spec.layers) and spec.layers[2].ffn is None
    assert spec.layers[0].ffn.params["activation_constants"] == {"alpha": 1.702, "limit": 0.7, "shift": 1.0}
    assert spec.embedding.params["scale"] == 3.0 and spec.head.params["scale"] == 0.5
    assert spec.stream_parts[0][1].params["passes"] == 3
    # the tensors are those that the plain implementation draws, shape by shape
    w = plain.random_weights(MIXED, 0)
    specs = spec.weight_specs()
    assert set(specs) == set(w)
    assert all(tuple(specs[k].shape) == tuple(w[k].shape) for k in w)
    # no loop: every layer once, no table of pass vectors
    flat = copy.deepcopy(MIXED)
    del flat["loop"]
    spec = model_spec_for(config_from_dict(flat))
    assert [r.layer for r in spec.schedule] == [0, 1, 2, 3] and not spec.stream_parts and "loop.step" not in spec.weight_specs()


def test_the_cache_each_mixer_asks_for():
    from torchless_rs_amd.parts.base import make_part
    spec = model_spec_for(config_from_dict(copy.deepcopy(MIXED)))
    a = make_part("mixer", spec.layers[0].mixer).kv_request()
    assert (a.n_kv_heads, a.head_dim, a.window, a.v_head_dim) == (2, 16, 20, 8)
    b = make_part("mixer", spec.layers[1].mixer).kv_request()          # the two maps of a key side by side
    assert (b.n_kv_heads, b.head_dim, b.window, b.v_head_dim) == (2, 16, None, 24)
    d = make_part("mixer", spec.layers[3].mixer).kv_request()          # values as wide as both maps: one width
    assert (d.n_kv_heads, d.head_dim, d.v_head_dim) == (2, 32, None)


# ---- the plain implementation's mechanisms, each against a property that pins it ------------------

def test_plain_sink_takes_weight_without_a_value():
    s = torch.zeros(1, 3, 3, dtype=torch.float64)
    a = plain.softmax_with_sink(s, plain.visible(3), torch.tensor([0.0], dtype=torch.float64))
    assert torch.allclose(a[0].sum(-1), torch.tensor([1 / 2, 2 / 3, 3 / 4], dtype=torch.float64))
    big = plain.softmax_with_sink(s, plain.visible(3), torch.tensor([50.0], dtype=torch.float64))
    assert float(big.sum()) < 1e-20


def test_plain_window_and_rotation():
    ok = plain.visible(6, 3)
    assert ok[5].tolist() == [False, False, False, True, True, True] and ok[1].tolist() == [True, True] + [False] * 4
    assert plain.visible(4, 1).int().tolist() == torch.eye(4).int().tolist()
    t = torch.randn(5, 2, 10, dtype=torch.float64)
    r = plain.rotate(t, torch.arange(5), 100.0, 6)
    assert torch.equal(r[..., 6:], t[..., 6:]) and torch.equal(r[0], t[0])
    assert torch.allclose((r[..., :6] ** 2).sum(-1), (t[..., :6] ** 2).sum(-1))
    # a dot product of two rotated units depends on the distance alone
    a, b = torch.randn(1, 1, 10, dtype=torch.float64), torch.randn(1, 1, 10, dtype=torch.float64)
    d1 = (plain.rotate(a, torch.tensor([7]), 100.0, 6) * plain.rotate(b, torch.tensor([3]), 100.0, 6)).sum()
    d2 = (plain.rotate(a, torch.tensor([14]), 100.0, 6) * plain.rotate(b, torch.tensor([10]), 100.0, 6)).sum()
    assert abs(float(d1 - d2)) < 1e-9


def test_plain_difference_of_equal_maps_and_the_clamp():
    w = {"p.lq1": torch.zeros(4, dtype=torch.float64), "p.lk1": torch.zeros(4, dtype=torch.float64),
         "p.lq2": torch.ones(4, dtype=torch.float64), "p.lk2": torch.full((4,), 0.25, dtype=torch.float64)}
    assert plain.diff_lambda(w, "p.", 0.3) == pytest.approx(1.0 - math.e + 0.3)
    h = torch.tensor([[10.0, -10.0]], dtype=torch.float64)
    w = {"f.gate": torch.eye(2, dtype=torch.float64), "f.up": torch.eye(2, dtype=torch.float64),
         "f.down": torch.eye(2, dtype=torch.float64)}
    y = plain.clamped_feed_forward(h, w, "f.", {"limit": 2.0})
    g0, g1 = 2.0, -10.0                       # the gate is clamped from above only, up on both sides
    want = [g0 / (1 + math.exp(-1.702 * g0)) * 3.0, g1 / (1 + math.exp(-1.702 * g1)) * -1.0]
    assert y[0].tolist() == pytest.approx(want)


def test_plain_passes_add_the_embedding_again():
    cfg = copy.deepcopy(MIXED)
    w = plain.random_weights(cfg, 5)
    ids = [3, 50, 7, 7, 100]
    streams = []
    plain.forward(w, cfg, ids, streams)
    assert len(streams) == 8
    one = copy.deepcopy(cfg)
    one["loop"]["times"] = 1
    w1 = dict(w)
    w1["loop.step"] = w["loop.step"][:1]
    s1 = []
    plain.forward(w1, one, ids, s1)
    assert len(s1) == 4 and torch.equal(s1[2], streams[2]) and not torch.equal(s1[3], streams[3])
