"""Configuration, plan and cache bookkeeping of the Metitar decoder, and the plain implementation against itself
(no GPU)."""

import copy
import math

import pytest
import torch

from metitar_helpers import METITAR
from plain import metitar_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.cache.pool import CacheError
from somi_inference_amd.config import ConfigError, MetitarConfig, config_from_dict
from somi_inference_amd.models import collect_weight_specs, metitar_plan
from somi_inference_amd.models.decoder import DecoderModel
from somi_inference_amd.parts import BorrowedCache, CompositeSpec, FixedStateSpec, PagedSpec, Runtime
from somi_inference_amd.parts.position import RotaryPosition


@pytest.mark.parametrize("name", list(METITAR))
def test_config_round_trips_through_its_json(name):
    config = METITAR[name]["config"]
    raw = config.to_dict()
    assert raw["architecture"] == "Metitar"
    arch, again = config_from_dict(copy.deepcopy(raw))
    assert arch.name == "Metitar" and again == config and isinstance(again, MetitarConfig)


def test_keys_a_config_may_leave_out():
    raw = METITAR["A"]["config"].to_dict()
    del raw["token_side"], raw["embedding"], raw["logit_scale"], raw["canon"]
    del raw["layers"][1]["mlp"]["shared"], raw["layers"][0]["mixer"]["rot"]["scaling"], raw["layers"][2]["mixer"]["rot"]["scaling"]
    raw["layers"][0]["mlp"] = None
    _, config = config_from_dict(raw)
    assert config.token_side_dim is None and config.canon_taps is None
    assert config.embedding_scale == 1.0 and config.logit_scale == 1.0
    assert config.layers[1].mlp.shared_ff is None and config.layers[0].mixer.rot_scaling is None
    names = {spec.name for spec in collect_weight_specs(metitar_plan(config))}
    assert "side.embed" not in names and "l0.canon1" not in names and "l1.mlp.shared.gate" not in names
    assert "l0.mlp.up" not in names and "l0.norm2" not in names and "l1.mlp.e7.down" in names


def test_config_errors_name_the_key():
    raw = METITAR["A"]["config"].to_dict()
    for change, text in (
        (lambda r: r["layers"][0].__setitem__("type", "attention"), "'type'"),
        (lambda r: r["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda r: r["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
        (lambda r: r["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "rot.dims"),
        (lambda r: r["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
        (lambda r: r["layers"][2]["mixer"].__setitem__("kv_from", 2), "kv_from"),
        (lambda r: r["layers"][2]["mixer"].__setitem__("kv_rank", 16), "kv_rank"),
        (lambda r: r["layers"][1]["mlp"]["router"].__setitem__("top", 9), "top"),
        (lambda r: r["layers"][1]["mlp"].__setitem__("kind", "sparse"), "kind"),
        (lambda r: r["layers"][1]["mixer"].pop("vdim"), "vdim"),
        (lambda r: r.pop("width"), "width"),
    ):
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(broken)


def test_plan_names_tensors_and_borrowed_caches():
    config = METITAR["A"]["config"]
    plan = metitar_plan(config)
    names = {spec.name: spec for spec in collect_weight_specs(plan)}
    assert {"embed", "side.embed", "head", "final.norm", "final.norm.b", "l0.norm1.b", "l0.canon1", "l0.mix.dq.norm",
            "l0.mix.dkv", "l0.mix.sink", "l0.mlp.act", "l1.mix.f.b", "l1.mix.lower", "l1.mlp.e7.up", "l1.mlp.router",
            "l2.mlp.shared.down", "l3.side.norm"} <= set(names)
    assert "l2.mix.dkv" not in names and "l2.mix.dkv.norm" not in names       # the borrower projects no latent
    assert "l3.norm2" not in names and "l3.mlp.up" not in names               # a layer without a feed-forward
    assert names["l0.mix.uq"].shape == (4 * (16 + 16), 40) and names["l0.mix.dkv"].shape == (32 + 16, 96)
    assert names["l2.mix.uk"].shape == (2 * 24, 32) and names["l0.canon1"].shape == (96, 3)
    assert names["side.embed"].shape == (211, 4 * 8) and not any(name.endswith(".weight") for name in names)
    model = DecoderModel(plan, Runtime(torch.float32, torch.device("cpu")))
    needs = model.cache_needs()
    assert all(isinstance(need, CompositeSpec) for need in needs)
    own, borrowed = dict(needs[0].parts), dict(needs[2].parts)
    assert isinstance(own["mixer"], PagedSpec) and [t.name for t in own["mixer"].tensors] == ["latent", "latent_t"]
    assert [t.elements_per_token() for t in own["mixer"].tensors] == [32 + 16, 32] and own["mixer"].window is None
    assert own["input"] == FixedStateSpec((2, 96), torch.float32)
    assert borrowed["mixer"] == BorrowedCache(0, ("mixer",)) and isinstance(borrowed["input"], FixedStateSpec)
    assert dict(needs[1].parts)["mixer"] == FixedStateSpec((3, 16, 24), torch.float32)
    cache = CacheManager(needs, block_size=16, num_blocks=8, max_requests=2, dtype=torch.float32, device="cpu")
    lender, reader = cache.layer_caches[0].children["mixer"], cache.layer_caches[2].children["mixer"]
    assert reader.tensors["latent"] is lender.tensors["latent"] and lender.writes and not reader.writes
    assert cache.layer_caches[2].children["input"].state is not cache.layer_caches[0].children["input"].state
    assert len(cache.groups) == 1 and cache.groups[0].runs == [0]
    # every layer's kept rows and both recurrent states are cleared for a new request; the borrowed pages are nobody's state
    assert len(cache.state_caches()) == 4 + 2
    cache.register("a")
    cache.reserve("a", 70)
    cache.commit("a", 70)
    cache.check_invariants()
    cache.free("a")
    assert cache.free_pages() == [8]
    # without an input convolution the borrower's need is the lender's run itself
    raw = config.to_dict()
    del raw["canon"]
    needs = DecoderModel(metitar_plan(config_from_dict(raw)[1]), Runtime(torch.float32, torch.device("cpu"))).cache_needs()
    assert needs[2] == 0 and isinstance(needs[0], PagedSpec) and isinstance(needs[1], FixedStateSpec)


def test_a_part_of_a_composite_can_only_be_borrowed_from_an_earlier_run():
    spec = PagedSpec((__import__("somi_inference_amd").parts.PageTensor("t", ("page", 4)),))
    with pytest.raises(CacheError, match="earlier"):
        CacheManager([CompositeSpec((("mixer", BorrowedCache(1, ("mixer",))),)), CompositeSpec((("mixer", spec),))],
                     block_size=4, num_blocks=4, max_requests=1, dtype=torch.float32, device="cpu", allocate_tensors=False)
    with pytest.raises(CacheError, match="has none"):
        CacheManager([CompositeSpec((("mixer", spec),)), CompositeSpec((("mixer", BorrowedCache(0, ("other",))),))],
                     block_size=4, num_blocks=4, max_requests=1, dtype=torch.float32, device="cpu", allocate_tensors=False)


@pytest.mark.parametrize("dims,base,factor,original,fast,slow", [(16, 5000.0, 4.0, 64, 16.0, 2.0), (32, 1000.0, 8.0, 16, 64.0, 0.01),
                                                                 (8, 100.0, 3.0, 4096, 1.0, 0.5), (2, 10.0, 2.0, 8, 2.0, 1.0)])
def test_ramped_frequencies_against_the_formula(dims, base, factor, original, fast, slow):
    rot = {"dims": dims, "base": base, "scaling": {"factor": factor, "original": original, "fast": fast, "slow": slow}}
    want, amplitude = plain.rotary_frequencies(rot)
    part = RotaryPosition("", head_dim=dims, theta=base, rotary_dim=dims, scaling=rot["scaling"])
    torch.testing.assert_close(part.frequencies().double(), want, rtol=1e-6, atol=0.0)
    assert part.amplitude == pytest.approx(0.1 * math.log(factor) + 1.0) == pytest.approx(amplitude)
    plain_part = RotaryPosition("", head_dim=dims, theta=base, rotary_dim=dims)
    assert plain_part.amplitude == 1.0


# ------------------------------------------------------------------------------- the plain implementation against itself
def test_plain_recurrence_and_convolution_cut_in_two_equal_the_whole():
    """The plain functions hold whole sequences; the recurrence and the convolution carried over a cut by hand give
    the same, which is what the engine's state slots have to do."""
    gen = torch.Generator().manual_seed(3)
    h = torch.randn(19, 24, generator=gen, dtype=torch.float64)
    taps = torch.randn(24, 4, generator=gen, dtype=torch.float64)
    whole = plain.input_convolution(h, taps)
    for cut in (1, 2, 3, 7):
        padded = torch.cat([h[max(0, cut - 3):cut], h[cut:]])
        second = plain.input_convolution(padded, taps)[min(cut, 3):]
        # the first rows of the padded part lack their own past, the rows after the cut do not
        torch.testing.assert_close(second, whole[cut:]) if cut >= 3 else None
    mixer = {"heads": 2, "dim": 6, "vdim": 5}
    w = {"m.q": torch.randn(12, 24, generator=gen, dtype=torch.float64), "m.f": torch.randn(12, 24, generator=gen, dtype=torch.float64),
         "m.f.b": torch.randn(12, generator=gen, dtype=torch.float64), "m.lower": torch.rand(12, generator=gen, dtype=torch.float64),
         "m.v": torch.randn(10, 24, generator=gen, dtype=torch.float64), "m.norm": torch.ones(5, dtype=torch.float64),
         "m.o": torch.randn(24, 10, generator=gen, dtype=torch.float64)}
    out = plain.hgrn2(h, w, "m", mixer, 1e-6)
    assert out.shape == (19, 24) and bool(torch.isfinite(out).all())
    # the first token: S = (1 - f) v^T, so the normed head is v / rms(v) times the sign of (1 - f) . q
    q = plain.silu(h[:1] @ w["m.q"].T).view(2, 6)
    f = (w["m.lower"] + (1 - w["m.lower"]) * torch.sigmoid(h[:1] @ w["m.f"].T + w["m.f.b"])).view(2, 6)
    v = (h[:1] @ w["m.v"].T).view(2, 5)
    first = plain.rms(v * ((1 - f) * q).sum(-1, keepdim=True), 1e-6).reshape(1, 10) @ w["m.o"].T
    torch.testing.assert_close(out[:1], first)


def test_plain_router_takes_the_largest_scores_as_they_are():
    weights = {"r.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [-1.0, 0.0], [0.5, 0.5]])}
    h = torch.tensor([[2.0, 0.0], [0.0, -3.0]])
    chosen, weight, margin = plain.routing(h, weights, "r", {"router": {"top": 2}})
    assert chosen.tolist() == [[0, 3], [0, 2]]            # equal scores: the lower index first
    torch.testing.assert_close(weight, torch.sigmoid(torch.tensor([[2.0, 1.0], [0.0, 0.0]])))
    assert float(margin[0]) > 0.2 and float(margin[1]) == pytest.approx(0.5 - float(torch.sigmoid(torch.tensor(-1.5))))
