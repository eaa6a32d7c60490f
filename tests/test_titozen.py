"""The Titozen architecture without a GPU: its configuration, the model's tensors and caches, and the cache manager's
handling of a block that keeps a state slot beside windowed pages."""
import copy

import pytest
import torch

from ginfer_amd import config_from_dict
from ginfer_amd.cache import CacheManager
from ginfer_amd.config import ConfigError
from ginfer_amd.parts import PagedSpec, StateSpec
from ginfer_amd.parts.model import build_model

CFG = dict(architecture="Titozen", vocab=97, width=40, norm=dict(eps=2e-6), canon=dict(taps=3), layers=[
    dict(type="hgrn2", mixer=dict(heads=2, dim=12, vdim=20), mlp=dict(kind="dense", ff=56, limit=1.25)),
    dict(type="latent_attention", mixer=dict(heads=3, dim=8, vdim=16, q_rank=24, kv_rank=10, scale=0.3, mask=dict(size=21)),
         mlp=None),
    dict(type="hgrn2", mixer=dict(heads=1, dim=5, vdim=7), mlp=None),
])


def test_configuration_reads_every_size_and_round_trips():
    cfg = config_from_dict(CFG)
    assert type(cfg).__name__ == "TitozenConfig" and cfg.to_dict() == CFG
    assert config_from_dict(cfg.to_dict()).to_dict() == CFG
    spec = cfg.model_spec()
    assert [l.parts["mixer"].kind for l in spec.layers] == ["hgrn2", "latent_attention", "hgrn2"]
    assert "feed_forward" in spec.layers[0].parts and "feed_forward" not in spec.layers[1].parts
    la = spec.layers[1].parts["mixer"].params
    assert (la["num_heads"], la["head_dim"], la["value_dim"], la["q_rank"], la["kv_rank"], la["scale"], la["window"]) == \
        (3, 8, 16, 24, 10, 0.3, 21)
    assert spec.layers[0].parts["feed_forward"].params["limit"] == 1.25
    assert spec.layers[0].parts["input_conv"].params["taps"] == 3 and spec.final_norm.params["eps"] == 2e-6


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("canon"), "canon"),
    (lambda c: c["layers"][0].update(type="lstm"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "feed-forward kind"),
    (lambda c: c["layers"][0]["mixer"].update(heads=0), "heads"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_configuration_errors_name_the_key(change, word):
    c = copy.deepcopy(CFG)
    change(c)
    with pytest.raises(ConfigError, match=word):
        config_from_dict(c)


def test_tensor_names_shapes_and_caches():
    model = build_model(config_from_dict(CFG).model_spec(), torch.float32, None)
    shapes = {n: tuple(s.shape) for n, s in model.weight_specs().items()}
    assert shapes["embed"] == (97, 40) and shapes["embed.norm"] == () and shapes["final.norm"] == () and shapes["head"] == (97, 40)
    assert shapes["l0.canon1"] == (40, 3) and shapes["l0.norm1"] == () and shapes["l0.norm2"] == ()
    assert shapes["l0.mix.q"] == (24, 40) and shapes["l0.mix.f.b"] == (24,) and shapes["l0.mix.lower"] == (24,)
    assert shapes["l0.mix.v"] == (40, 40) and shapes["l0.mix.norm"] == (20,) and shapes["l0.mix.o"] == (40, 40)
    assert shapes["l0.mlp.gate"] == (56, 40) and shapes["l0.mlp.down"] == (40, 56)
    assert shapes["l1.mix.dq"] == (24, 40) and shapes["l1.mix.uq"] == (24, 24) and shapes["l1.mix.dkv.norm"] == (10,)
    assert shapes["l1.mix.uk"] == (24, 10) and shapes["l1.mix.uv"] == (48, 10) and shapes["l1.mix.sink"] == (3,)
    assert shapes["l1.mix.g"] == (3, 40) and shapes["l1.mix.o"] == (40, 48)
    assert "l1.norm2" not in shapes and "l1.mlp.gate" not in shapes and "l2.norm2" not in shapes
    specs = model.cache_specs()
    assert specs[0] == [StateSpec((2, 40)), StateSpec((2, 12, 20))]
    assert specs[1] == [StateSpec((2, 40)), PagedSpec((("c", 10),), 21)]          # 32-bit: the latent alone
    half = build_model(config_from_dict(CFG).model_spec(), torch.bfloat16, None).cache_specs()
    assert half[1][1] == PagedSpec((("c", 10),), 21)                              # a rank that is no multiple of 8
    c = copy.deepcopy(CFG)
    c["layers"][1]["mixer"]["kv_rank"] = 16
    half = build_model(config_from_dict(c).model_spec(), torch.bfloat16, None).cache_specs()
    assert half[1][1] == PagedSpec((("c", 16), ("ct", 16)), 21)                   # bfloat16: and its transposed copy
    assert model.capturable()


def test_a_layer_without_a_mask_sees_every_earlier_position():
    c = copy.deepcopy(CFG)
    del c["layers"][1]["mixer"]["mask"]
    spec = config_from_dict(c).model_spec()
    assert spec.layers[1].parts["mixer"].params["window"] is None
    model = build_model(spec, torch.float32, None)
    assert model.cache_specs()[1][1] == PagedSpec((("c", 10),), None)


def test_one_tap_keeps_no_convolution_state():
    c = copy.deepcopy(CFG)
    c["canon"]["taps"] = 1
    model = build_model(config_from_dict(c).model_spec(), torch.float32, None)
    assert model.cache_specs()[0][0] is None and model.cache_specs()[1][0] is None


def test_random_draws_of_the_lower_bounds_lie_inside_the_unit_interval(tmp_path):
    from ginfer_amd import write_random_model
    from safetensors.torch import load_file
    folder = write_random_model(str(tmp_path / "m"), config_from_dict(CFG), seed=1, dtype="bfloat16", std_scale=5.0)
    t = load_file(folder + "/model.safetensors")
    lower = t["l0.mix.lower"].float()
    assert float(lower.min()) >= 1 / 64 and float(lower.max()) <= 63 / 64 and float(lower.std()) > 0.05
    assert t["l0.norm1"].shape == () and t["embed.norm"].shape == ()


def test_cache_manager_gives_slots_and_windowed_pages_back():
    """State slots beside windowed pages: a request's pages behind the window return to the pool while it runs, its slot
    and the rest when it ends, and the next request takes both over."""
    specs = build_model(config_from_dict(CFG).model_spec(), torch.float32, None).cache_specs()
    cm = CacheManager(specs, page_size=8, num_pages=6, max_requests=2)
    assert len(cm.groups) == 1 and cm.groups[0].window == 21 and len(cm.state_units) == 5
    cm.admit("a")
    cm.admit("b")
    assert not cm.can_admit()
    slot_a = cm.slot("a")
    for _ in range(10):                          # 80 tokens through a pool of 48: only the window's pages are held
        cm.append("a", 8)
        cm.commit("a")
        cm.check()
    held = [p for p in cm.table("a", 0) if p >= 0]
    assert cm.length("a") == 80 and len(held) <= CacheManager.window_span_pages(21, 8)
    cm.append("b", 5)
    cm.commit("b")
    cm.release("a")
    cm.admit("c")
    assert cm.slot("c") == slot_a and cm.length("c") == 0
    cm.append("c", 30)
    cm.commit("c")
    cm.check()
    cm.release("b")
    cm.release("c")
    cm.check()
    assert cm.groups[0].pool.num_free == 6
