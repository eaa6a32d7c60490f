"""The Potupel architecture without a GPU: its configuration, the order of runs with the loop's re-entries, the model's
tensors and caches, the rescaled rotary frequencies, and the plain statement's own mechanisms against hand-made cases."""
import copy
import math

import pytest
import torch

import plain_potupel as pp
from ginfer_amd import config_from_dict
from ginfer_amd.cache import CacheManager
from ginfer_amd.config import ConfigError
from ginfer_amd.parts import KVCacheSpec, StateSpec
from ginfer_amd.parts.model import build_model
from ginfer_amd.parts.rope import RotaryNeoX

ROT = dict(base=5000.0, dims=8, scaling=dict(factor=4.0, low=1.0, high=3.0, original=64))
CFG = dict(architecture="Potupel", vocab=101, width=48, norm=dict(eps=2e-6), loop=dict(start=1, stop=3, times=2), layers=[
    dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.3, conv=3, rot=ROT),
         mlp=dict(kind="dense", ff=56)),
    dict(type="attention", mixer=dict(heads=3, kv_heads=3, dim=16, vdim=8, scale=0.2, conv=2, rot=dict(base=100.0, dims=16)),
         mlp=dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=24), shared=dict(ff=40))),
    dict(type="attention", mixer=dict(heads=2, kv_heads=1, dim=8, vdim=8, scale=0.5), mlp=None),
    dict(type="attention", mixer=dict(heads=1, kv_heads=1, dim=32, vdim=16, scale=0.1, conv=5, rot=dict(base=10.0, dims=2)),
         mlp=dict(kind="moe", router=dict(experts=3, top=3), expert=dict(ff=16))),
])


def test_configuration_reads_every_size_and_round_trips():
    cfg = config_from_dict(CFG)
    assert type(cfg).__name__ == "PotupelConfig" and cfg.to_dict() == CFG
    spec = cfg.model_spec()
    assert [l.arrangement for l in spec.layers] == ["sandwich"] * 4
    m0 = spec.layers[0].parts["mixer"].params
    assert (m0["num_heads"], m0["num_kv_heads"], m0["head_dim"], m0["value_dim"], m0["scale"], m0["taps"], m0["sink"]) == \
        (4, 2, 12, 20, 0.3, 3, 0.0)
    assert m0["position"].params["scaling"] == ROT["scaling"] and m0["position"].params["rotary_dim"] == 8
    assert spec.layers[1].parts["mixer"].params["position"].params["scaling"] is None
    assert spec.layers[2].parts["mixer"].params["position"] is None and spec.layers[2].parts["mixer"].params["taps"] is None
    assert "feed_forward" not in spec.layers[2].parts and "feed_forward_out_norm" not in spec.layers[2].parts
    assert spec.layers[0].parts["feed_forward"].kind == "squared_relu"
    ff = spec.layers[1].parts["feed_forward"].params
    assert (ff["num_experts"], ff["top_k"], ff["expert_size"], ff["shared_size"]) == (5, 2, 24, 40)
    assert spec.layers[3].parts["feed_forward"].params["shared_size"] is None
    assert spec.final_norm.params["eps"] == 2e-6 and spec.final_norm.params["gain_offset"] == 1.0 and spec.head.params["tied"]


def test_the_loop_orders_the_runs_and_marks_where_passes_start():
    spec = config_from_dict(CFG).model_spec()
    assert [(e.layer, e.enter) for e in spec.schedule] == [(0, ()), (1, (0,)), (2, ()), (1, (1,)), (2, ()), (3, ())]
    assert spec.reentry.params["passes"] == 2 and spec.tail_enter == ()
    assert pp.layer_runs(CFG) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    c = copy.deepcopy(CFG)
    c.pop("loop")
    spec = config_from_dict(c).model_spec()
    assert [(e.layer, e.enter) for e in spec.schedule] == [(i, ()) for i in range(4)] and spec.reentry is None
    c["loop"] = dict(start=0, stop=4, times=1)
    assert [(e.layer, e.enter) for e in config_from_dict(c).model_spec().schedule] == [(0, (0,)), (1, ()), (2, ()), (3, ())]
    c["loop"] = dict(start=4, stop=4, times=2)           # a loop without layers at the end: its passes start behind the last run
    assert config_from_dict(c).model_spec().tail_enter == (0, 1)


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][0].update(type="lstm"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_heads"), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "feed-forward kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=14), "dims"),
    (lambda c: c["loop"].update(stop=9), "loop"),
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
    assert shapes["embed"] == (101, 48) and shapes["final.norm"] == (48,) and "head" not in shapes and "head.weight" not in shapes
    assert shapes["loop.in"] == (48, 96) and shapes["loop.step"] == (2, 48)
    for n in ("norm1", "norm1b", "norm2", "norm2b", "ls1", "ls2"):
        assert shapes["l0." + n] == (48,)
    assert "l2.norm2" not in shapes and "l2.ls2" not in shapes and shapes["l2.ls1"] == (48,)
    assert shapes["l0.mix.q"] == (48, 48) and shapes["l0.mix.k"] == (24, 48) and shapes["l0.mix.v"] == (40, 48)
    assert shapes["l0.mix.o"] == (48, 80) and shapes["l0.mix.q.conv"] == (48, 3) and shapes["l0.mix.v.conv"] == (40, 3)
    assert "l2.mix.q.conv" not in shapes
    assert shapes["l0.mlp.up"] == (56, 48) and shapes["l0.mlp.down"] == (48, 56)
    assert shapes["l1.mlp.router"] == (5, 48) and shapes["l1.mlp.router.b"] == (5,)
    assert shapes["l1.mlp.e4.gate"] == (24, 48) and shapes["l1.mlp.e0.down"] == (48, 24) and shapes["l1.mlp.shared.up"] == (40, 48)
    assert "l3.mlp.shared.up" not in shapes and "l1.mlp.e5.gate" not in shapes
    specs = model.cache_specs()
    assert len(specs) == 6
    state, kv = specs[0]
    assert isinstance(state, StateSpec) and state.shape[0] == 2 and isinstance(kv, KVCacheSpec) and kv.num_kv_heads == 2
    assert specs[2][0] is None                          # no convolution: no state
    assert specs[1] == specs[3] and specs[1][0].shape[0] == 1      # the two passes keep caches of their own, of one kind


def test_cache_manager_gives_every_run_of_a_looped_layer_its_own_cache():
    model = build_model(config_from_dict(CFG).model_spec(), torch.float32, None)
    cm = CacheManager(model.cache_specs(), page_size=8, num_pages=6, max_requests=2)
    cm.admit("a")
    cm.append("a", 20)
    cm.commit("a")
    cm.admit("b")
    assert cm.can_append("b", 24) and not cm.can_append("b", 25)
    cm.release("a")
    assert cm.can_append("b", 48)
    cm.check()
    owners = {cm.group_of[(i, 1)] for i in range(6)}
    assert len(owners) == 6                              # six runs, six places, although two layers run twice


def test_rescaled_frequencies_follow_the_wavelength_rule():
    part = RotaryNeoX(theta=5000.0, rotary_dim=8, max_positions=64, scaling=ROT["scaling"])
    got = part._wide_frequencies(4)
    want = pp.rotary_frequencies(ROT)
    assert torch.equal(got, want)
    plainf = [5000.0 ** (-2.0 * i / 8) for i in range(4)]
    lengths = [2 * math.pi / f for f in plainf]
    kinds = ["kept" if l < 64 / 3.0 else "divided" if l > 64 / 1.0 else "blended" for l in lengths]
    assert set(kinds) == {"kept", "divided", "blended"}          # the test's constants reach all three branches
    for f, g, kind in zip(plainf, got.tolist(), kinds):
        if kind == "kept":
            assert abs(g - f) < 1e-6 * f
        elif kind == "divided":
            assert abs(g - f / 4.0) < 1e-6 * f
        else:
            assert f / 4.0 < g < f
    cos, sin = RotaryNeoX(theta=5000.0, rotary_dim=8, max_positions=64, scaling=ROT["scaling"], device="cpu").tables()
    ang = torch.arange(64, dtype=torch.float32)[:, None] * want[None, :]
    assert torch.allclose(cos, torch.cos(ang)) and torch.allclose(sin, torch.sin(ang))


def test_plain_mechanisms_on_hand_made_cases():
    # convolution: zeros before the start, the last tap on the token itself
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=torch.float64)
    w = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)
    assert pp.channel_convolution(u, w).flatten().tolist() == [1.0, 12.0, 124.0]
    # the sink: one key with score 0 gets half of the weight, the sink the other half
    q = torch.zeros((1, 4), dtype=torch.float64)
    v = torch.tensor([[3.0, 5.0]], dtype=torch.float64)
    assert pp.sink_softmax_attention(q, q.clone(), v, 1, 1, 4, 2, 1.0).tolist() == [[1.5, 2.5]]
    # routing: the two largest, softmax over them alone
    w = {"r.router": torch.eye(3, dtype=torch.float64), "r.router.b": torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64)}
    ids, weights = pp.route(torch.tensor([[2.0, 0.5, 0.0]], dtype=torch.float64), w, "r", 3, 2)
    assert ids.tolist() == [[0, 2]] and abs(float(weights[0, 0]) - 1 / (1 + math.exp(-1.0))) < 1e-12
    # rotation: a quarter turn swaps the pair
    rot = dict(base=1.0, dims=2)
    x = torch.tensor([[0.0, 0.0, 7.0], [1.0, 0.0, 7.0]], dtype=torch.float64)
    got = pp.rotate(x, 1, 3, rot)
    assert torch.allclose(got[1], torch.tensor([math.cos(1.0), math.sin(1.0), 7.0], dtype=torch.float64), atol=1e-7)
