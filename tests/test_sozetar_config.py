"""The Sozetar configuration, its registry entry, tensor names and cache requests (no GPU)."""
import copy
import json

import pytest
import torch

import plain_sozetar as plain
from torchless_rs_amd.config import ConfigError, SozetarConfig, config_from_dict, load_config
from torchless_rs_amd.models import model_spec_for


def att(heads, kv_heads, dim, vdim, scale, window=None, temp=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def layer(mixer, ff=None):
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# layers that differ in every size; a reader that looks further back than the owner; a layer without feed-forward
MIXED = {"architecture": "Sozetar", "vocab": 160, "width": 64, "norm": {"eps": 1e-5}, "layers": [
    layer(att(4, 2, 16, 32, 0.3, window=5, temp=(0.5, 3)), ff=48),
    layer(att(4, 2, 16, 32, 0.2, window=9, kv_from=0)),
    layer(att(2, 1, 24, 8, 0.25), ff=96),
    layer(att(8, 2, 16, 32, 0.3, window=3, temp=(0.1, 7), kv_from=0), ff=40),
]}


def test_every_key_is_read():
    c = config_from_dict(copy.deepcopy(MIXED))
    assert isinstance(c, SozetarConfig)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, len(c.layers)) == (160, 64, 1e-5, 4)
    m0, m1, m2, m3 = (l.mixer for l in c.layers)
    assert (m0.heads, m0.kv_heads, m0.dim, m0.vdim, m0.scale, m0.window) == (4, 2, 16, 32, 0.3, 5)
    assert (m0.q_temp_coef, m0.q_temp_every, m0.kv_from) == (0.5, 3.0, None)
    assert (m1.window, m1.kv_from, m1.q_temp_coef) == (9, 0, None)
    assert (m2.window, m2.heads, m2.vdim) == (None, 2, 8)
    assert (m3.heads, m3.kv_from) == (8, 0)
    assert [l.ff for l in c.layers] == [48, None, 96, 40]


def test_defaults_and_round_trip():
    d = copy.deepcopy(MIXED)
    del d["layers"][2]["mixer"]["kv_heads"], d["layers"][2]["mixer"]["vdim"]
    c = config_from_dict(d)
    assert c.layers[2].mixer.kv_heads == 2 and c.layers[2].mixer.vdim == 24
    assert config_from_dict(c.to_dict()) == c
    assert config_from_dict(json.loads(json.dumps(c.to_dict()))) == c


@pytest.mark.parametrize("path, value, word", [
    (("vocab",), None, "vocab"),
    (("width",), 0, "width"),
    (("norm",), None, "norm"),
    (("layers",), [], "layers"),
    (("layers", 0, "type"), "recurrent", "type"),
    (("layers", 0, "mixer", "heads"), 3, "multiple"),
    (("layers", 0, "mixer", "dim"), 300, "up to 256"),
    (("layers", 0, "mixer", "scale"), None, "scale"),
    (("layers", 0, "mixer", "mask"), {"size": 0}, "size"),
    (("layers", 0, "mixer", "q_temp"), {"coef": 0.1, "every": 0}, "every"),
    (("layers", 1, "mixer", "kv_from"), 1, "earlier"),
    (("layers", 3, "mixer", "kv_from"), 1, "none of its own"),
    (("layers", 1, "mixer", "dim"), 32, "differ"),
    (("layers", 0, "mlp"), {"kind": "routed", "ff": 8}, "kind"),
])
def test_errors(path, value, word):
    d = copy.deepcopy(MIXED)
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        config_from_dict(d)
    assert word in str(e.value)


def test_tensor_names_and_shapes_follow_the_configuration():
    spec = model_spec_for(config_from_dict(copy.deepcopy(MIXED)))
    got = {k: tuple(v.shape) for k, v in spec.weight_specs().items()}
    assert got == plain.tensor_shapes(MIXED)
    assert "l1.mix.k" not in got and "l1.norm2" not in got and "l3.mix.v.b" not in got
    assert [r.kv_from for r in spec.schedule] == [None, 0, None, 0]


def test_a_model_folder_written_and_read(tmp_path):
    from torchless_rs_amd import write_random_model
    from util import read_model_dir
    d = write_random_model(str(tmp_path / "m"), copy.deepcopy(MIXED), seed=3, std=0.1, norm_std=0.1)
    c = load_config(d)
    assert c == config_from_dict(copy.deepcopy(MIXED))
    cfg, tensors = read_model_dir(d)
    assert cfg["architecture"] == "Sozetar"
    assert {k: tuple(v.shape) for k, v in tensors.items()} == plain.tensor_shapes(MIXED)
    assert float(tensors["l0.mix.o.b"].float().abs().max()) > 0       # biases are drawn, not zero


def test_the_owner_of_keys_keeps_what_its_farthest_reader_needs():
    from torchless_rs_amd.engine.model import Model
    from torchless_rs_amd.cache.cache import NO_RING
    d = copy.deepcopy(MIXED)
    d["layers"][0]["mixer"]["mask"]["size"] = 70
    d["layers"][1]["mixer"]["mask"]["size"] = 130       # the reader looks back over three pages
    m = Model(model_spec_for(config_from_dict(d)), None, torch.float32, "cpu")
    kv, _ = m.cache_requests()
    assert sorted(kv) == [0, 2] and kv[0].window == 130 and kv[0].v_head_dim == 32
    cache = m.make_cache(64 * 16, allocate=False)
    runs = m.bind_cache(cache)
    assert runs[1].kv_group is runs[0].kv_group and runs[3].kv_layer == runs[0].kv_layer
    assert runs[0].kv_group.ring_pages == 3 and runs[2].kv_group.ring_pages == NO_RING
    assert runs[0].kv_read_later and not runs[2].kv_read_later and not runs[1].kv_owner
    del d["layers"][3]["mixer"]["mask"]                 # a reader without a window: the owner keeps everything
    m = Model(model_spec_for(config_from_dict(d)), None, torch.float32, "cpu")
    assert m.cache_requests()[0][0].window is None


def test_the_plain_mechanisms_on_values_worked_by_hand():
    # layer norm of (1, 2, 3, 6): mean 3, variance 3.5
    y = plain.layer_norm(torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=torch.float64), torch.ones(4, dtype=torch.float64), 0.0)
    assert torch.allclose(y, torch.tensor([[-2.0, -1.0, 0.0, 3.0]], dtype=torch.float64) / 3.5 ** 0.5)
    # the factor on q steps up at positions every - 1, 2 every - 1, ...
    t = plain.query_temperature(7, 0.5, 3)
    assert torch.allclose(t[:2], torch.ones(2, dtype=torch.float64)) and float(t[2]) == pytest.approx(1 + 0.5 * 0.6931471805599453)
    assert float(t[5]) == pytest.approx(1 + 0.5 * 1.0986122886681098) and float(t[4]) == float(t[2])
    assert plain.head_slopes(4).tolist() == pytest.approx([0.25, 0.0625, 0.015625, 0.00390625])
    v = plain.visible(5, 2)
    assert v[3].tolist() == [False, False, True, True, False] and plain.visible(3, None)[2].all()
    # one key, score 0, sink 0: the key gets half of the weight
    o = plain.attend(torch.zeros(1, 1, 2, dtype=torch.float64), torch.ones(1, 1, 2, dtype=torch.float64),
                     torch.tensor([[[4.0, 8.0]]], dtype=torch.float64), 1.0, None, torch.zeros(1, dtype=torch.float64), None)
    assert o.flatten().tolist() == pytest.approx([2.0, 4.0])
    assert float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) == pytest.approx(0.8411919906082768)
