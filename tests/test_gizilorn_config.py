"""The Gizilorn configuration, its plan and what the plan asks of the cache manager (no GPU)."""

import copy

import pytest

from gizilorn_helpers import GIZILORN
from somi_inference_amd.config import ConfigError, GizilornConfig, config_from_dict
from somi_inference_amd.models import DecoderModel, collect_weight_specs, gizilorn_plan
from somi_inference_amd.parts import Runtime

import torch


def raw(name="A"):
    return GIZILORN[name]["config"].to_dict()


@pytest.mark.parametrize("name", list(GIZILORN))
def test_config_round_trip_and_registry(name):
    config = GIZILORN[name]["config"]
    arch, again = config_from_dict(config.to_dict())
    assert arch.name == "Gizilorn" and again == config
    assert isinstance(again, GizilornConfig)


def test_keys_a_model_may_leave_out():
    data = raw("A")
    del data["layers"][2]["mixer"]["softcap"], data["layers"][2]["mixer"]["mask"], data["streams"]
    config = GizilornConfig.from_dict(data)
    assert config.layers[2].mixer.softcap is None and config.layers[2].mixer.window is None and config.streams is None
    assert config.layers[1].mlp is None and config.layers[3].mixer.window is None


@pytest.mark.parametrize("change,word", [
    (lambda d: d["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda d: d["layers"][2]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda d: d["layers"][2]["mixer"]["rot"].update(dims=33), "rot.dims"),
    (lambda d: d["layers"][2]["mixer"].update(vdim=15), "vdim"),
    (lambda d: d["layers"][1]["mixer"].update(kv_from=2), "kv_from"),
    (lambda d: d["layers"][1]["mixer"].update(kv_from=1), "kv_from"),
    (lambda d: d["layers"][1]["mixer"].update(kv_rank=48), "kv_rank"),
    (lambda d: d["layers"][0].update(type="recurrence"), "type"),
    (lambda d: d["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda d: d.update(streams=0), "streams"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), "size"),
])
def test_what_is_refused(change, word):
    data = copy.deepcopy(raw("A"))
    change(data)
    with pytest.raises(ConfigError, match=word):
        GizilornConfig.from_dict(data)


def test_tensor_names_and_shapes():
    specs = {s.name: s for s in collect_weight_specs(gizilorn_plan(GIZILORN["A"]["config"]))}
    assert specs["embed"].shape == (301, 96) and specs["embed.norm"].shape == (96,) and specs["final.norm"].shape == (96,)
    assert specs["l0.mix.q"].shape == (4 * 24, 96) and specs["l0.mix.dkv"].shape == (48, 96)
    assert specs["l0.mix.dkv.norm"].shape == (40,) and specs["l0.mix.g"].shape == (96, 96)
    assert specs["l0.mix.uk"].shape == (64, 40) and specs["l0.mix.uv"].shape == (96, 40)
    assert "l1.mix.dkv" not in specs and "l1.mix.dkv.norm" not in specs and "l1.mlp.up" not in specs
    assert "l1.hc2.in" not in specs and specs["l1.hc1.mix"].shape == (3, 3) and specs["l0.hc2.out"].shape == (3,)
    assert specs["l2.mix.q.b"].shape == (128,) and specs["l2.mix.k"].shape == (64, 96) and specs["l2.mix.v.b"].shape == (32,)
    assert specs["l2.mix.talk"].shape == (4, 4) and specs["l2.mix.o"].shape == (96, 64)
    assert specs["l2.mlp.up.b"].shape == (80,) and specs["l2.mlp.act"].shape == (2,) and specs["l2.mlp.down.b"].shape == (96,)
    assert not any(name.endswith(".weight") or name.endswith(".bias") for name in specs)
    plain_sum = {s.name for s in collect_weight_specs(gizilorn_plan(GIZILORN["C"]["config"]))}
    assert not any(".hc" in name for name in plain_sum)
    one_stream = {s.name: s for s in collect_weight_specs(gizilorn_plan(GIZILORN["B"]["config"]))}
    assert one_stream["l0.hc1.mix"].shape == (1, 1)


def test_a_lender_keeps_rows_for_its_farthest_seeing_reader():
    model = DecoderModel(gizilorn_plan(GIZILORN["A"]["config"]), Runtime(torch.float32, torch.device("cpu")))
    needs = model.cache_needs()
    assert needs[0].window == 33 and needs[1] == 0          # layer 0 sees 20 keys, its reader 33
    assert needs[2].window == 12 and needs[3].window is None
    assert model.layers[0].mixer.window == 20 and model.layers[1].mixer.window == 33
    model = DecoderModel(gizilorn_plan(GIZILORN["C"]["config"]), Runtime(torch.float32, torch.device("cpu")))
    needs = model.cache_needs()
    assert needs[0].window == 11 and needs[2] == 0 and needs[3] == 0
    data = raw("C")
    del data["layers"][3]["mixer"]["mask"]                   # a reader that sees everything: rows are kept for ever
    model = DecoderModel(gizilorn_plan(GizilornConfig.from_dict(data)), Runtime(torch.float32, torch.device("cpu")))
    assert model.cache_needs()[0].window is None


def test_connection_tensors_are_what_the_checkpoint_says_for_one_stream():
    one = GIZILORN["B"]["config"]                       # streams = 1
    assert one.fitted_to({"l0.hc1.in": (1,), "l0.mix.q": (48, 64)}) is one
    assert one.fitted_to({"l0.mix.q": (48, 64)}).streams is None
    none = GIZILORN["C"]["config"]                      # no key
    assert none.fitted_to({"l0.mix.q": (16, 80)}) is none
    assert none.fitted_to({"l0.hc1.in": (2,), "l0.hc1.mix": (2, 2)}).streams == 2
    three = GIZILORN["A"]["config"]
    assert three.fitted_to({"l0.mix.q": (1, 1)}) is three          # three streams need their tensors: the loader says so
