"""Each mechanism of the Metitar decoder alone: the part with its kernels and the engine's cache manager against the
plain function written from the equations."""

import math

import pytest
import torch

from plain import metitar_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine.batch import StepEntry, build_step
from somi_inference_amd.kernels import ops
from somi_inference_amd.parts import CompositeSpec, PartSpec, Runtime, build_part

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = torch.device("cuda:0")


def tol(dtype, loose=1.0):
    return dict(rtol=1e-4, atol=2e-5 * loose) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2 * loose)


def check(got, want, dtype, loose=1.0):
    """float32: element by element.  bfloat16: the error against the size of what is compared, since sums of some
    hundred rounded products are off by a share of their size: its root mean square within 2 % of the values' and no
    element off by more than 8 % of the largest."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape and bool(torch.isfinite(got).all())
    if dtype == torch.float32:
        size = max(1.0, float(want.pow(2).mean().sqrt()))         # sums of many products are off by a share of their size
        torch.testing.assert_close(got, want, rtol=1e-4, atol=2e-5 * loose * size)
        return
    error = got - want
    assert float(error.pow(2).mean().sqrt()) <= 0.02 * float(want.pow(2).mean().sqrt()) + 1e-3, \
        f"root mean square error {float(error.pow(2).mean().sqrt()):.3e} of values of {float(want.pow(2).mean().sqrt()):.3e}"
    assert float(error.abs().max()) <= 0.08 * float(want.abs().max()) + 1e-3, \
        f"largest error {float(error.abs().max()):.3e} of values up to {float(want.abs().max()):.3e}"


def rounded(x: torch.Tensor, dtype) -> torch.Tensor:
    """float32 values that the dtype holds exactly, so that the kernel and the plain function start from the same."""
    return x.to(dtype).to(torch.float32)


def load_part(part, weights: dict, dtype):
    """Hand the part its tensors as the loader would: matrices in the compute dtype, vectors in float32."""
    roles = {spec.name: spec.role for spec in part.weight_specs()}
    assert set(roles) == set(weights), sorted(set(roles) ^ set(weights))
    part.load(lambda name: weights[name].to(dtype if roles[name] == "matrix" else torch.float32).to(DEV).contiguous(),
              Runtime(dtype, DEV))
    return part


def random_weights(part, dtype, seed, scale=None) -> dict:
    """float32 tensors for every tensor the part declares (all hold values bfloat16 has exactly)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for spec in part.weight_specs():
        value = torch.randn(spec.shape, generator=gen) * (scale or {}).get(spec.role, spec.init.std * (10 if spec.role == "matrix" else 1))
        out[spec.name] = rounded(value + spec.init.mean, torch.bfloat16)
    return out


class Engine:
    """The cache manager and the step layout of the engine around one mixer (or one input convolution)."""

    def __init__(self, mixer, dtype, block_size, num_blocks=64, max_requests=4, spec=None):
        self.mixer, self.dtype = mixer, dtype
        self.cache = CacheManager([spec or mixer.cache_spec()], block_size=block_size, num_blocks=num_blocks,
                                  max_requests=max_requests, dtype=dtype, device=DEV)

    def run(self, portions, in_dtype=None):
        """One step of (request, its next input rows); the part's output rows per request."""
        entries = []
        for rid, x in portions:
            if not self.cache.has(rid):
                self.cache.register(rid)
            self.cache.reserve(rid, x.shape[0])
            entries.append(StepEntry(rid, [0] * x.shape[0], []))
        step = build_step(entries, self.cache, DEV, () if getattr(self.mixer, 'entry_split', None) is None else (self.mixer.entry_split,))
        y = self.mixer.forward(torch.cat([x for _, x in portions]).to(in_dtype or self.dtype).to(DEV).contiguous(), step,
                               self.cache.layer_caches[0])
        for rid, x in portions:
            self.cache.commit(rid, x.shape[0])
        outs, at = [], 0
        for _, x in portions:
            outs.append(y[at:at + x.shape[0]].float().cpu())
            at += x.shape[0]
        return outs

    def run_cut(self, rid, x, sizes, in_dtype=None):
        outs, at, i = [], 0, 0
        while at < x.shape[0]:
            size = sizes[i % len(sizes)]
            outs.append(self.run([(rid, x[at:at + size])], in_dtype)[0])
            at += size
            i += 1
        self.cache.free(rid)
        return torch.cat(outs)


# ------------------------------------------------------------------------------------------ layer norm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [7, 96, 1000])
def test_layer_norm_and_its_add_into_the_stream(dtype, width):
    gen = torch.Generator().manual_seed(width)
    norm = build_part("norm", PartSpec("layer_norm", {"hidden_size": width, "eps": 1e-5, "tensor": "n"}), prefix="")
    w = {"n": rounded(torch.randn(width, generator=gen), torch.bfloat16), "n.b": rounded(torch.randn(width, generator=gen), torch.bfloat16)}
    load_part(norm, w, dtype)
    # rows with a large common offset: the variance must come from the deviations
    h = torch.randn(9, width, generator=gen) + torch.tensor([0.0, 100.0, -3.0, 0.0, 1e3, 0.0, 5.0, 0.0, 0.0])[:, None]
    want = plain.layer_norm(h, w, "n", 1e-5)
    got = norm.forward(h.to(DEV)).float().cpu()
    torch.testing.assert_close(got, want, **(dict(rtol=1e-3, atol=2e-3) if dtype == torch.float32 else tol(dtype, 3)))
    y = rounded(torch.randn(9, width, generator=gen) * 5, dtype)
    for copy in (None, dtype):
        stream = h.clone().to(DEV)
        rows = norm.add_normed(stream, y.to(dtype).to(DEV), copy)
        torch.testing.assert_close(stream.cpu(), h + plain.layer_norm(y, w, "n", 1e-5), rtol=1e-5, atol=2e-4)
        assert (rows is None) == (copy is None)
        if rows is not None:
            assert rows.dtype == dtype and torch.equal(rows.float().cpu(), stream.cpu().to(dtype).float())


# ------------------------------------------------------------------------------------------ the input convolution
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,width", [(1, 24), (2, 100), (4, 96), (5, 300), (9, 8), (17, 40)])
def test_input_convolution_whole_cut_and_side_by_side(dtype, taps, width):
    gen = torch.Generator().manual_seed(taps)
    conv = build_part("input_conv", PartSpec("short_causal", {"hidden_size": width, "taps": taps}), prefix="c")
    w = {"c": rounded(torch.randn(width, taps, generator=gen) * 0.5, torch.bfloat16)}
    load_part(conv, w, dtype)
    x = torch.randn(37, width, generator=gen)
    want = plain.input_convolution(x, w["c"])
    engine = Engine(conv, dtype, 8, spec=conv.state_spec())
    whole = engine.run_cut("a", x, [37], torch.float32)
    torch.testing.assert_close(whole, want, **tol(dtype))
    for sizes in ([1], [2], [3, 1, 1, 7], [taps, 1], [20, 2, 15]):       # portions shorter than the taps shift the kept rows
        assert torch.equal(engine.run_cut("a", x, sizes, torch.float32), whole), f"portions of {sizes}"
    other = torch.randn(11, width, generator=gen)
    a1, b1 = engine.run([("a", x[:5]), ("b", other[:9])], torch.float32)
    b2, a2 = engine.run([("b", other[9:]), ("a", x[5:])], torch.float32)
    assert torch.equal(torch.cat([a1, a2]), whole)
    torch.testing.assert_close(torch.cat([b1, b2]), plain.input_convolution(other, w["c"]), **tol(dtype))


# ------------------------------------------------------------------------------------------ latent attention
def latent_mixer(dtype, heads, dim, rot, vdim, rank, q_rank, scale, page, width=64, dims=None, scaling=None, shares=False,
                 seed=1, base=50.0):
    dims = rot if dims is None else dims
    position = PartSpec("rotary", {"head_dim": rot, "theta": base, "rotary_dim": dims, "pairing": "half", "scaling": scaling}) \
        if dims else PartSpec("none", {})
    part = build_part("mixer", PartSpec("latent_attention", {
        "hidden_size": width, "num_heads": heads, "dim": dim, "rot_dim": rot, "value_dim": vdim, "kv_rank": rank,
        "q_rank": q_rank, "scale": scale, "eps": 1e-5, "position": position, "shares_cache": shares, "page_size": page,
        "suffix": ""}), prefix="m")
    weights = random_weights(part, dtype, seed, {"matrix": 0.3})
    config = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank, "scale": scale,
              "rot": {"base": base, "dims": dims, **({"scaling": scaling} if scaling else {})}}
    return load_part(part, weights, dtype), weights, config


def plain_latent(x, weights, config, kept=None):
    kept = kept if kept is not None else plain.latent_keys(x, weights, "m", config, 1e-5)
    return plain.latent_attention(x, weights, "m", config, 1e-5, kept)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,vdim,rank,q_rank,page,dims,scaling", [
    (4, 16, 8, 24, 32, 40, 16, None, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}),
    (1, 8, 2, 8, 16, 8, 4, None, None),
    (5, 12, 6, 20, 28, 20, 8, 2, None),
    (2, 64, 32, 48, 160, 72, 16, None, {"factor": 8.0, "original": 16, "fast": 64.0, "slow": 0.01}),
    (3, 24, 0, 8, 48, 16, 8, None, None),
    (16, 32, 16, 32, 64, 48, 16, None, None),
    (8, 128, 64, 128, 512, 96, 16, None, None),
    (20, 16, 16, 16, 48, 32, 8, None, None),              # more heads than a workgroup's 16 query slots
    (37, 8, 8, 8, 24, 16, 16, 4, None),
    (2, 16, 16, 16, 656, 32, 16, None, None),              # a latent wider than the matrix-core kernel takes
])
def test_latent_attention_against_the_plain_function(dtype, heads, dim, rot, vdim, rank, q_rank, page, dims, scaling):
    mixer, weights, config = latent_mixer(dtype, heads, dim, rot, vdim, rank, q_rank, (dim + rot) ** -0.5, page, dims=dims,
                                          scaling=scaling)
    tokens = 45 if rank > 256 else 83
    x = rounded(torch.randn(tokens, 64, generator=torch.Generator().manual_seed(7)), dtype)
    want = plain_latent(x, weights, config)
    engine = Engine(mixer, dtype, page)
    whole = engine.run_cut("a", x, [tokens])
    check(whole, want, dtype, 4)
    for sizes in ([1], [2], [5, 1, 1, 17], [page, page + 1], [40, 3]):
        got = engine.run_cut("a", x, sizes)
        check(got, want, dtype, 4)
        if dtype == torch.float32:
            assert torch.equal(got, whole), f"float32 results depend on the portions {sizes}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sink", [-30.0, 0.0, 6.0, 40.0])
def test_the_sink_stands_in_the_denominator_only(dtype, sink):
    """A sink far below the scores changes nothing; one far above them takes nearly all the weight, so the output
    nearly vanishes; it is not multiplied by the scale."""
    mixer, weights, config = latent_mixer(dtype, 2, 16, 8, 16, 32, 24, 0.05, 8)
    weights["m.sink"] = torch.tensor([sink, sink / 2])
    load_part(mixer, weights, dtype)
    x = rounded(torch.randn(30, 64, generator=torch.Generator().manual_seed(8)), dtype)
    got = Engine(mixer, dtype, 8).run_cut("a", x, [13, 1, 16])
    want = plain_latent(x, weights, config)
    check(got, want, dtype, 4)
    if sink == 40.0:
        assert float(got.abs().max()) < 1e-3 * float(x.abs().max()) * 64


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far,page,decoded", [(0, 8, False), (0, 16, True), (7, 8, True), (8, 8, False), (15, 16, True),
                                               (16, 16, False), (127, 16, True), (128, 16, False), (129, 16, True), (300, 16, True),
                                               (407, 16, False), (419, 16, True)])
def test_one_far_key_stands_out(dtype, far, page, decoded):
    """The kept vector at position ``far`` (the first token, either side of a page border or of a 128-key tile, the
    query's own neighbourhood) is made to match the last query, up to hundreds of tokens later, much better than any
    other: the output is then that vector.  The query arrives alone (a decoded token) or as the last of a portion."""
    tokens, count = 420, (1 if decoded else 12)
    mixer, weights, config = latent_mixer(dtype, 2, 16, 16, 16, 32, 24, 1.0, page, seed=far + 1)
    x = rounded(torch.randn(tokens, 64, generator=torch.Generator().manual_seed(far)) * 0.2, dtype)
    engine = Engine(mixer, dtype, page)
    engine.run([("a", x[:tokens - count])])
    engine.cache.reserve("a", count)
    step = build_step([StepEntry("a", [0] * count, [])], engine.cache, DEV, mixer_splits(mixer))
    cache, cache_t = (engine.cache.layer_caches[0].tensors[name] for name in ("latent", "latent_t"))
    rows = torch.tensor(engine.cache.slots(0, "a", 0, tokens), device=DEV)

    def keep(position, vector):
        """Put a vector where the layer would have kept it: the row, and the latent part transposed inside its page."""
        slot = int(rows[position])
        cache.view(-1, 48)[slot] = vector.to(dtype).to(DEV)
        cache_t[slot // page, :, slot % page] = vector[:32].to(dtype).to(DEV)
    fresh = torch.randn(count, 48, generator=torch.Generator().manual_seed(1)) * 0.1
    for i in range(count):
        keep(tokens - count + i, fresh[i])
    marked = torch.zeros(48)
    marked[5], marked[20] = 6.0, -3.0
    keep(far, marked)
    queries = torch.zeros(count, 2, 48)
    queries[:, :, 5] = 8.0                                   # the query's part on the latent's side points along channel 5
    queries[:, 1, 33] = 0.5
    got = mixer.attend(queries.to(dtype).to(DEV), cache, step, step.paged[0], cache_t).float().cpu()
    kept = cache.view(-1, 48)[rows].float().cpu()
    scores = torch.einsum("hr,tr->ht", queries[0], kept)
    share = torch.softmax(torch.cat([scores, weights["m.sink"][:, None]], dim=1), dim=1)
    assert float(share[:, far].min()) > 0.9, "the marked key does not stand out in this test's own arithmetic"
    want = share[:, :-1] @ kept[:, :32]
    check(got[-1], want, dtype, 2)
    assert float((got[-1, :, 5] - 6.0).abs().max()) < 0.7
    if far < tokens - count:                                 # every row of the portion sees it
        assert float((got[:, :, 5] - 6.0).abs().max()) < 0.7


def mixer_splits(mixer):
    return () if mixer.entry_split is None else (mixer.entry_split,)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_layer_reads_the_latents_another_layer_kept(dtype):
    """Two mixers in one plan position each: the second has no projection of its own latent and reads the first's pages
    with its own maps, queries and sinks."""
    lender, w1, c1 = latent_mixer(dtype, 3, 16, 8, 24, 32, 40, 0.2, 8, seed=3)
    reader, w2, c2 = latent_mixer(dtype, 5, 8, 8, 16, 32, 16, 0.3, 8, seed=4, shares=True)
    assert "m.dkv" not in w2 and "m.dkv" in w1
    cache = CacheManager([lender.cache_spec(), 0], block_size=8, num_blocks=32, max_requests=2, dtype=dtype, device=DEV)
    gen = torch.Generator().manual_seed(5)
    x1, x2 = (rounded(torch.randn(50, 64, generator=gen), dtype) for _ in range(2))
    got = []
    cache.register("a")
    for start, count in ((0, 20), (20, 1), (21, 29)):
        cache.reserve("a", count)
        step = build_step([StepEntry("a", [0] * count, [])], cache, DEV, mixer_splits(lender))
        lender.forward(x1[start:start + count].to(dtype).to(DEV), step, cache.layer_caches[0])
        got.append(reader.forward(x2[start:start + count].to(dtype).to(DEV), step, cache.layer_caches[1]).float().cpu())
        cache.commit("a", count)
    kept = plain.latent_keys(x1, w1, "m", c1, 1e-5)
    if dtype == torch.bfloat16:
        kept = tuple(rounded(t, dtype) for t in kept)
    check(torch.cat(got), plain_latent(x2, w2, c2, kept), dtype, 4)
    with pytest.raises(ValueError, match="not both"):
        reader.forward(x2[:1].to(dtype).to(DEV), step, cache.layer_caches[0])


# ------------------------------------------------------------------------------------------ HGRN2
def hgrn2_mixer(dtype, heads, dim, vdim, seed=1, width=64):
    part = build_part("mixer", PartSpec("hgrn2", {"hidden_size": width, "num_heads": heads, "key_dim": dim, "value_dim": vdim,
                                                  "eps": 1e-5, "suffix": ""}), prefix="m")
    weights = random_weights(part, dtype, seed, {"matrix": 0.3})
    weights["m.lower"] = rounded(torch.rand(heads * dim, generator=torch.Generator().manual_seed(seed)) * 0.9, torch.bfloat16)
    return load_part(part, weights, dtype), weights, {"heads": heads, "dim": dim, "vdim": vdim}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 16, 24), (1, 24, 40), (5, 12, 20), (1, 128, 64), (2, 7, 5), (4, 64, 128)])
def test_hgrn2_against_the_plain_function(dtype, heads, dim, vdim):
    mixer, weights, config = hgrn2_mixer(dtype, heads, dim, vdim)
    x = rounded(torch.randn(90, 64, generator=torch.Generator().manual_seed(dim)), dtype)
    want = plain.hgrn2(x, weights, "m", config, 1e-5)
    engine = Engine(mixer, dtype, 8)
    whole = engine.run_cut("a", x, [90])
    check(whole, want, dtype, 6)
    for sizes in ([1], [2], [7, 1, 1, 30], [16, 17]):           # prompts against token-by-token decoding and portions
        got = engine.run_cut("a", x, sizes)
        assert torch.equal(got, whole) if dtype == torch.float32 else True
        check(got, want, dtype, 6)


def test_hgrn2_gate_bounds_and_two_requests_side_by_side():
    """A lower bound of one keeps the state as it is and writes nothing (the output is zero from an empty state); a
    gate far open forgets everything but the current token.  Two requests in one step keep their own state."""
    dtype = torch.float32
    mixer, weights, config = hgrn2_mixer(dtype, 2, 16, 8)
    x = rounded(torch.randn(20, 64, generator=torch.Generator().manual_seed(2)), dtype)
    frozen = dict(weights, **{"m.lower": torch.ones(32)})
    load_part(mixer, frozen, dtype)
    out = Engine(mixer, dtype, 8).run_cut("a", x, [20])
    torch.testing.assert_close(out, plain.hgrn2(x, frozen, "m", config, 1e-5), **tol(dtype))
    opened = dict(weights, **{"m.lower": torch.zeros(32), "m.f.b": torch.full((32,), -40.0)})
    load_part(mixer, opened, dtype)
    out = Engine(mixer, dtype, 8).run_cut("a", x, [20])
    torch.testing.assert_close(out, plain.hgrn2(x, opened, "m", config, 1e-5), **tol(dtype))
    torch.testing.assert_close(out[7:8], plain.hgrn2(x[7:8], opened, "m", config, 1e-5), **tol(dtype))    # no memory at all
    load_part(mixer, weights, dtype)
    engine = Engine(mixer, dtype, 8)
    other = rounded(torch.randn(15, 64, generator=torch.Generator().manual_seed(3)), dtype)
    a1, b1 = engine.run([("a", x[:9]), ("b", other[:1])])
    b2, a2 = engine.run([("b", other[1:]), ("a", x[9:])])
    torch.testing.assert_close(torch.cat([a1, a2]), plain.hgrn2(x, weights, "m", config, 1e-5), **tol(dtype))
    torch.testing.assert_close(torch.cat([b1, b2]), plain.hgrn2(other, weights, "m", config, 1e-5), **tol(dtype))


# ------------------------------------------------------------------------------------------ feed-forwards
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,tokens", [(64, 80, 5), (100, 36, 70), (96, 304, 300)])
def test_normed_power_feed_forward_against_the_plain_function(dtype, width, ff, tokens):
    part = build_part("feed_forward", PartSpec("poly_norm", {"hidden_size": width, "intermediate_size": ff, "eps": 1e-5,
                                                            "suffix": ""}), prefix="f")
    weights = random_weights(part, dtype, ff, {"matrix": 0.3})
    weights["f.act"] = torch.tensor([0.5, -0.25, 0.125, 0.75])
    load_part(part, weights, dtype)
    x = rounded(torch.randn(tokens, width, generator=torch.Generator().manual_seed(1)), dtype)
    got = part.forward(x.to(dtype).to(DEV)).float().cpu()
    check(got, plain.poly_norm_ff(x, weights, "f", 1e-5), dtype, 8)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,ff,shared,tokens", [(8, 2, 32, 48, 40), (5, 1, 40, None, 3), (3, 3, 24, 8, 150),
                                                          (16, 4, 64, 64, 700), (4, 2, 9, None, 17)])
def test_sigmoid_scored_experts_weigh_their_inputs(dtype, experts, top, ff, shared, tokens):
    width = 72
    part = build_part("feed_forward", PartSpec("routed_experts", {
        "hidden_size": width, "num_experts": experts, "top": top, "expert_size": ff, "limit": None, "alpha": 1.0, "shift": 0.0,
        "shared_size": shared, "scores": "sigmoid", "normalize": False, "weight_on": "input", "suffix": ""}), prefix="f")
    weights = random_weights(part, dtype, experts, {"matrix": 0.25})
    weights["f.router"] = rounded(torch.randn(experts, width, generator=torch.Generator().manual_seed(9)) * 0.5, torch.bfloat16)
    load_part(part, weights, dtype)
    x = rounded(torch.randn(tokens, width, generator=torch.Generator().manual_seed(2)), dtype)
    mlp = {"router": {"experts": experts, "top": top}, **({"shared": {"ff": shared}} if shared else {})}
    chosen, weight, margin = plain.routing(x, weights, "f", mlp)
    got_chosen, got_weight = ops.moe_route(x.to(dtype).to(DEV), part.router, top, 1, 1, "sigmoid", False)
    sure = margin > 1e-4
    assert torch.equal(got_chosen.cpu()[sure].sort(dim=1).values, chosen[sure].sort(dim=1).values.int())
    torch.testing.assert_close(got_weight.cpu()[sure].sort(dim=1).values, weight[sure].sort(dim=1).values, rtol=1e-5, atol=1e-6)
    got = part.forward(x.to(dtype).to(DEV)).float().cpu()
    want = plain.routed_experts(x, weights, "f", mlp)
    check(got[sure], want[sure], dtype, 8)
    # the weight is on the input, where the unit is not linear: weighing the outputs instead gives something else
    scaled = torch.zeros_like(want)
    for t in range(min(tokens, 20)):
        for e, w in zip(chosen[t].tolist(), weight[t]):
            scaled[t] += w * plain.gated_unit(x[t:t + 1], weights, f"f.e{e}")[0]
    if shared:
        scaled += plain.gated_unit(x, weights, "f.shared")
    assert float((scaled[:min(tokens, 20)] - want[:min(tokens, 20)]).abs().max()) > 1e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pads", [(5, 3), (8, 4)])          # strides the matrix-core kernel refuses, and ones it takes
@pytest.mark.parametrize("heads,n_out,k,rows", [(3, 32, 16, 5), (1, 7, 9, 1), (6, 96, 32, 130), (2, 160, 64, 33), (16, 512, 128, 70),
                                                (4, 48, 104, 64)])
def test_per_head_products(dtype, pads, heads, n_out, k, rows):
    gen = torch.Generator().manual_seed(rows)
    x = rounded(torch.randn(rows, heads, k + pads[0], generator=gen), dtype)
    w = rounded(torch.randn(heads, n_out, k, generator=gen), dtype)
    out = torch.zeros(rows, heads, n_out + pads[1], dtype=dtype, device=DEV)
    ops.head_linear(x.to(dtype).to(DEV)[:, :, :k], w.to(dtype).to(DEV), out=out[:, :, :n_out])
    want = torch.einsum("thk,hok->tho", x[:, :, :k], w)
    check(out[:, :, :n_out].float().cpu(), want, dtype, 8)
    assert float(out[:, :, n_out:].abs().max()) == 0.0


@pytest.mark.parametrize("lanes", [4, 16])
@pytest.mark.parametrize("heads,dim,vdim", [(2, 64, 32), (1, 128, 64), (3, 100, 20), (2, 16, 8), (1, 256, 12)])
def test_the_recurrence_with_either_number_of_lanes_a_column(lanes, heads, dim, vdim):
    """The recurrence kernel spreads a column of the state over 4 or over 16 lanes; both against the recurrence written
    out, from a state that is not empty, with two requests of unequal length in one launch."""
    gen = torch.Generator().manual_seed(dim + lanes)
    n = 37
    rows = torch.randn(n, 2 * heads * dim + heads * vdim, generator=gen)
    keep = torch.rand(n, heads * dim, generator=gen)
    state = torch.randn(3, heads, dim, vdim, generator=gen)
    starts = torch.tensor([0, 30, n], dtype=torch.int32)
    slots = torch.tensor([2, 0], dtype=torch.int32)
    qk = heads * dim
    device_rows, device_state = rows.to(DEV), state.clone().to(DEV)
    got = ops.gla_scan(device_rows[:, :qk], device_rows[:, qk:2 * qk], device_rows[:, 2 * qk:], keep.to(DEV), starts.to(DEV),
                       slots.to(DEV), device_state, 0.5, lanes=lanes).cpu()
    want = torch.zeros(n, heads, vdim)
    after = state.clone()
    for entry, slot in enumerate(slots.tolist()):
        s = after[slot]
        for t in range(int(starts[entry]), int(starts[entry + 1])):
            q, k = rows[t, :qk].view(heads, dim), rows[t, qk:2 * qk].view(heads, dim)
            v = rows[t, 2 * qk:].view(heads, vdim)
            s = keep[t].view(heads, dim, 1) * s + k[:, :, None] * v[:, None, :]
            want[t] = torch.einsum("hkv,hk->hv", s, q * 0.5)
        after[slot] = s
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(device_state.cpu(), after, rtol=1e-4, atol=1e-4)
