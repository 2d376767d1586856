"""Each mechanism of the Gizilorn decoder alone: the part with its kernels and the engine's cache manager against the
plain function written from the equations."""

import math

import pytest
import torch

from gizilorn_helpers import PartEngine, load_part, random_weights, rounded
from plain import gizilorn_plain as plain
from somi_inference_amd.kernels import ops
from somi_inference_amd.parts import PartSpec, ResidualStream, Runtime, build_part

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = torch.device("cuda:0")


def check(got, want, dtype, loose=1.0):
    """float32: element by element against the values' size.  bfloat16: the error's root mean square within 2 % of the
    values' and no element off by more than 8 % of the largest; a wrong key, page or edge moves rows by their own size."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape and bool(torch.isfinite(got).all())
    size = float(want.pow(2).mean().sqrt())
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-4, atol=3e-5 * loose * max(1.0, size))
        return
    error = got - want
    assert float(error.pow(2).mean().sqrt()) <= 0.02 * loose * size + 1e-3, \
        f"root mean square error {float(error.pow(2).mean().sqrt()):.3e} of values of {size:.3e}"
    assert float(error.abs().max()) <= 0.08 * loose * float(want.abs().max()) + 1e-3, \
        f"largest error {float(error.abs().max()):.3e} of values up to {float(want.abs().max()):.3e}"


# ------------------------------------------------------------------------------------------ the streams
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("streams,width,rows", [(1, 8, 3), (2, 100, 17), (3, 96, 5), (4, 1000, 9), (8, 260, 2), (3, 7, 4), (2, 1030, 3)])
def test_streams_read_write_and_both_in_one_launch(dtype, streams, width, rows):
    gen = torch.Generator().manual_seed(streams * width)
    lanes = torch.randn(streams, rows, width, generator=gen) * 3
    w = {"a.in": torch.randn(streams, generator=gen), "a.mix": torch.randn(streams, streams, generator=gen),
         "a.out": torch.randn(streams, generator=gen), "b.in": torch.randn(streams, generator=gen)}
    norm_w = torch.randn(width, generator=gen)
    y = rounded(torch.randn(rows, width, generator=gen) * 2, dtype)
    dev = {k: v.to(DEV) for k, v in w.items()}
    # read alone, with and without the norm
    u = plain.read_streams(lanes, w, "a.")
    got = ops.hc_step(lanes.to(DEV), read=True, in_weights=dev["a.in"])
    torch.testing.assert_close(got.cpu(), u, rtol=1e-5, atol=1e-5)
    got = ops.hc_step(lanes.to(DEV), read=True, in_weights=dev["a.in"], norm_weight=norm_w.to(DEV), eps=1e-6, out_dtype=dtype)
    check(got, plain.rms(u, 1e-6) * norm_w, dtype)
    # the plain sum, and a row fanned out
    torch.testing.assert_close(ops.hc_step(lanes.to(DEV), read=True).cpu(), lanes.sum(dim=0), rtol=1e-5, atol=1e-5)
    fanned = ops.hc_step(lanes[:1].contiguous().to(DEV), read=True, copies=streams)
    assert torch.equal(fanned.view(streams, rows, width).cpu(), lanes[:1].expand(streams, rows, width))
    # write alone, then write and the next read in one launch: every new stream comes from the OLD ones
    want = plain.write_streams(lanes, y, w, "a.")
    device_lanes = lanes.to(DEV)
    assert ops.hc_step(device_lanes, y=y.to(dtype).to(DEV), mix=dev["a.mix"], out_weights=dev["a.out"]) is None
    torch.testing.assert_close(device_lanes.cpu(), want, rtol=1e-5, atol=1e-4)
    device_lanes = lanes.to(DEV)
    nxt = ops.hc_step(device_lanes, y=y.to(dtype).to(DEV), mix=dev["a.mix"], out_weights=dev["a.out"], read=True,
                      in_weights=dev["b.in"], norm_weight=norm_w.to(DEV), eps=1e-6, out_dtype=dtype)
    torch.testing.assert_close(device_lanes.cpu(), want, rtol=1e-5, atol=1e-4)
    check(nxt, plain.rms(plain.read_streams(want, w, "b."), 1e-6) * norm_w, dtype)


def test_a_mix_that_swaps_streams_reads_the_old_ones():
    lanes = torch.stack([torch.full((2, 5), 1.0), torch.full((2, 5), 10.0)])
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    device_lanes = lanes.to(DEV)
    ops.hc_step(device_lanes, y=torch.zeros(2, 5, device=DEV), mix=swap.to(DEV), out_weights=torch.zeros(2, device=DEV))
    assert torch.equal(device_lanes.cpu(), lanes.flip(0))


def test_the_stream_object_fans_out_once_and_settles_to_the_sum():
    h = torch.randn(4, 12, device=DEV)
    stream = ResidualStream(h.clone())
    lanes = stream.fan_out(3)
    assert lanes.shape == (3, 4, 12) and all(torch.equal(lanes[s], h) for s in range(3))
    assert stream.fan_out(3) is lanes
    torch.testing.assert_close(stream.settle(), 3 * h)
    with pytest.raises(ValueError):
        stream.fan_out(2)
    with pytest.raises(RuntimeError):
        stream.add(h)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedded_rows_are_normed_in_float32(dtype):
    gen = torch.Generator().manual_seed(5)
    part = build_part("embedding", PartSpec("token_embedding", {"vocab_size": 50, "hidden_size": 36, "tensor": "embed",
                                                                "norm_tensor": "embed.norm", "norm_eps": 1e-3}), prefix="")
    w = {"embed": rounded(torch.randn(50, 36, generator=gen) * 0.01), "embed.norm": rounded(torch.randn(36, generator=gen))}
    load_part(part, w, dtype, DEV)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    got = part.forward(ids.to(DEV))
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), plain.rms(w["embed"][ids.long()], 1e-3) * w["embed.norm"], rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------------------------------ the feed-forward
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("numbers", [(0.0, 0.0), (-3.0, 2.0), (1.5, -4.0)])
def test_activation_on_both_sides_of_zero(dtype, numbers):
    z = torch.tensor([[-30.0, -5.0, -1.0, -1e-3, 0.0, 1e-3, 0.5, 2.0, 11.0]])
    pq = torch.tensor(numbers)
    got = ops.xielu(z.to(DEV), pq.to(DEV), dtype)
    check(got, plain.xielu(z, pq), dtype)
    if dtype == torch.float32:
        # at z = -30 two terms of size 15 nearly cancel: float32 leaves an absolute error of their rounding
        torch.testing.assert_close(got.cpu(), plain.xielu(z.double(), pq.double()).float(), rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,ff,rows", [(24, 40, 1), (96, 200, 7), (64, 328, 70)])
def test_dense_feed_forward_with_biases(dtype, width, ff, rows):
    part = build_part("feed_forward", PartSpec("activated", {"hidden_size": width, "intermediate_size": ff, "suffix": "",
                                                             "bias_suffix": "b"}), prefix="f")
    w = random_weights(part, ff, scale={"b": 0.5})
    load_part(part, w, dtype, DEV)
    x = rounded(torch.randn(rows, width, generator=torch.Generator().manual_seed(rows)), dtype)
    got = part.forward(x.to(dtype).to(DEV))
    got = got.materialize() if hasattr(got, "materialize") else got
    check(got, plain.dense(x, w, "f."), dtype)


# ------------------------------------------------------------------------------------------ attention with mixed heads
def mixed_part(heads, kv, dim, vdim, window, cap, rot_dims, base=1000.0, scale=None):
    position = PartSpec("rotary", {"head_dim": dim, "theta": base, "rotary_dim": rot_dims, "pairing": "half"})
    spec = PartSpec("mixed_heads_attention", {
        "hidden_size": 48, "num_heads": heads, "num_kv_heads": kv, "dim": dim, "value_dim": vdim, "position": position,
        "scale": scale if scale is not None else dim ** -0.5, "softcap": cap, "window": window, "sink_one": True,
        "head_mix": True, "value_rotation": {"theta": base, "pairing": "half"}, "qkv_bias": True, "suffix": "",
        "bias_suffix": "b"})
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "rot": {"base": base, "dims": rot_dims}}
    if cap:
        m["softcap"] = cap
    if window:
        m["mask"] = {"size": window}
    return build_part("mixer", spec, prefix="m"), m


def mixed_weights(part, seed, wide=3.0):
    w = random_weights(part, seed, scale={"q": 0.2 * wide, "k": 0.2 * wide, "v": 0.3, "o": 0.2, "b": 0.3, "talk": 0.3})
    w["m.talk"] = rounded(w["m.talk"] + torch.eye(w["m.talk"].shape[0]))
    return w


SIZES = [  # heads, kv, dim, vdim, window, cap, rot_dims, page
    (4, 2, 16, 16, 10, 12.0, 16, 8),
    (6, 6, 8, 24, None, None, 4, 4),
    (8, 2, 32, 8, 70, 30.0, 16, 16),
    (3, 1, 24, 40, 1, 5.0, 24, 8),
    (2, 2, 64, 64, 33, None, 32, 32),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dim,vdim,window,cap,rot_dims,page", SIZES)
def test_mixed_heads_attention_whole_cut_and_side_by_side(dtype, heads, kv, dim, vdim, window, cap, rot_dims, page):
    part, m = mixed_part(heads, kv, dim, vdim, window, cap, rot_dims)
    w = mixed_weights(part, heads * dim)
    load_part(part, w, dtype, DEV)
    gen = torch.Generator().manual_seed(dim)
    x = rounded(torch.randn(150, 48, generator=gen), dtype)
    other = rounded(torch.randn(37, 48, generator=gen), dtype)
    want, want_other = plain.attention(x, w, "m.", m), plain.attention(other, w, "m.", m)
    engine = PartEngine([part], dtype, DEV, page, num_blocks=64)
    whole = engine.run_cut("a", x, [150])[0]
    check(whole, want, dtype)
    for sizes in ([1], [2], [7, 1, 1, 30], [64, 3]):
        cut = engine.run_cut("a", x, sizes)[0]
        check(cut, want, dtype)
        if dtype == torch.float32:
            torch.testing.assert_close(cut, whole, rtol=2e-5, atol=2e-5)
    # two requests in the same steps, in pages that others have just given back
    got_a, got_b, at_a, at_b = [], [], 0, 0
    while at_a < 150 or at_b < 37:
        portions = []
        if at_a < 150:
            portions.append(("a", x[at_a:at_a + 13]))
        if at_b < 37:
            portions.append(("b", other[at_b:at_b + (1 if at_b > 5 else 3)]))
        outs = engine.run(portions)[0]
        if at_a < 150:
            got_a.append(outs[0])
            at_a += 13
        if at_b < 37:
            got_b.append(outs[-1])
            at_b += portions[-1][1].shape[0]
    check(torch.cat(got_a), want, dtype)
    check(torch.cat(got_b), want_other, dtype)
    engine.cache.free("a")
    engine.cache.free("b")
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page", [(9, 4), (16, 16), (65, 8), (130, 16)])
def test_a_marked_key_just_inside_and_just_outside_the_window(dtype, window, page):
    """One key is made to stand out for every query; the token whose window still holds it attends to it almost alone,
    the next token no longer sees it.  Prompts and single tokens."""
    part, m = mixed_part(2, 1, 16, 16, window, None, 0 + 2, base=1e6, scale=1.0)
    w = mixed_weights(part, window, wide=0.2)
    load_part(part, w, dtype, DEV)
    gen = torch.Generator().manual_seed(window)
    length, marked = window + 40, 21
    x = rounded(torch.randn(length, 48, generator=gen) * 0.3, dtype)
    # the marked token's input lies along a direction that the key matrix maps to a long key; every query carries a
    # constant part (its bias) along that key
    direction = torch.zeros(48)
    direction[5] = 1.0
    w["m.k"][:, 5] = 0.0
    w["m.k"][3, 5] = 8.0
    w["m.q.b"] = torch.zeros_like(w["m.q.b"])
    w["m.q.b"][3], w["m.q.b"][16 + 3] = 2.0, 2.0
    x[:, 5] = 0.0
    x[marked] = x[marked] + direction
    load_part(part, w, dtype, DEV)
    want = plain.attention(x, w, "m.", m)
    last_inside = marked + window - 1
    # the oracle itself shows the edge: the row that still sees the marked key differs from its neighbour's kind
    engine = PartEngine([part], dtype, DEV, page, num_blocks=64)
    for sizes in ([length], [last_inside, 1, 1, 1], [marked + 1, 1], [5, 2]):
        got = engine.run_cut("a", x, sizes)[0]
        check(got[marked:last_inside + 3], want[marked:last_inside + 3], dtype)
        check(got, want, dtype)
    without = x.clone()
    without[marked] = without[marked] - direction
    blind = plain.attention(without, w, "m.", m)
    assert float((want[last_inside] - blind[last_inside]).abs().max()) > 0.05       # seen by the last token inside
    if last_inside + 1 < length and window > 1:
        torch.testing.assert_close(want[last_inside + 1], blind[last_inside + 1], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_one_in_the_denominator_and_the_mix_each_matter(dtype):
    """A mix that swaps two heads swaps their weights but not their values' heads; with all scores 0 every key weighs
    1 / (1 + keys), the one being the sink's share."""
    part, m = mixed_part(2, 2, 8, 8, None, None, 8, scale=1.0)
    w = mixed_weights(part, 3)
    w["m.talk"] = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    load_part(part, w, dtype, DEV)
    x = rounded(torch.randn(20, 48, generator=torch.Generator().manual_seed(1)), dtype)
    engine = PartEngine([part], dtype, DEV, 8)
    check(engine.run_cut("a", x, [20])[0], plain.attention(x, w, "m.", m), dtype)
    w["m.q.b"] = torch.full_like(w["m.q.b"], 0.0)
    w["m.k.b"] = torch.full_like(w["m.k.b"], 0.0)
    w["m.q"] = rounded(w["m.q"] * 0 + 0.0)
    # all scores are 0: every key weighs 1 / (1 + keys), so the first token's output is half its value
    load_part(part, w, dtype, DEV)
    got = engine.run_cut("a", x, [20])[0]
    want = plain.attention(x, w, "m.", m)
    check(got, want, dtype)
    first_value = (x[:1] @ w["m.v"].T + w["m.v.b"]) @ w["m.o"].T
    torch.testing.assert_close(want[:1], 0.5 * first_value, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_of_rotated_values_far_from_the_start(dtype):
    """Values turned by positions in the hundreds and turned back by the query's: single tokens after a long prompt."""
    part, m = mixed_part(4, 2, 16, 32, 24, 25.0, 8, base=50.0)
    w = mixed_weights(part, 77)
    load_part(part, w, dtype, DEV)
    x = rounded(torch.randn(700, 48, generator=torch.Generator().manual_seed(9)), dtype)
    want = plain.attention(x, w, "m.", m)
    engine = PartEngine([part], dtype, DEV, 16, num_blocks=12)         # 192 tokens of pages: the window gives pages back
    got = engine.run_cut("a", x, [90] + [1] * 40 + [100])[0]
    check(got, want, dtype, loose=1.5)
    engine.cache.check_invariants()


# ------------------------------------------------------------------------------------------ latent attention
def latent_part(heads, dim, rot, vdim, rank, window, base=300.0, scale=None, shares=False, kept="same"):
    position = PartSpec("rotary", {"head_dim": rot, "theta": base, "rotary_dim": rot, "pairing": "neighbours"})
    spec = PartSpec("latent_attention", {
        "hidden_size": 48, "num_heads": heads, "dim": dim, "rot_dim": rot, "value_dim": vdim, "kv_rank": rank,
        "q_rank": None, "scale": scale if scale is not None else (dim + rot) ** -0.5, "eps": 1e-6, "position": position,
        "shares_cache": shares, "suffix": "", "sink": False, "window": window, "kept_window": kept, "gate": True})
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank,
         "scale": scale if scale is not None else (dim + rot) ** -0.5, "rot": {"base": base, "dims": rot}}
    if window:
        m["mask"] = {"size": window}
    return build_part("mixer", spec, prefix="m" if not shares else "n"), m


def latent_weights(part, seed, wide=3.0):
    return random_weights(part, seed, scale={"q": 0.2 * wide, "dkv": 0.3, "uk": 0.2 * wide, "uv": 0.3, "g": 0.3, "o": 0.2,
                                             "norm": 0.3})


LATENT_SIZES = [  # heads, dim, rot, vdim, rank, window, page
    (4, 16, 8, 24, 40, 20, 8),
    (2, 8, 4, 8, 24, None, 4),
    (3, 32, 16, 16, 48, 131, 16),
    (6, 16, 16, 32, 96, 7, 16),
    (1, 8, 2, 4, 16, 1, 8),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,vdim,rank,window,page", LATENT_SIZES)
def test_latent_attention_whole_cut_and_a_reader_of_its_cache(dtype, heads, dim, rot, vdim, rank, window, page):
    reader_window = None if window is None else window + 9
    part, m = latent_part(heads, dim, rot, vdim, rank, window, kept=reader_window)
    reader, m_reader = latent_part(heads + 1, dim // 2, rot, vdim, rank, reader_window, shares=True, scale=0.4)
    w, w_reader = latent_weights(part, rank), latent_weights(reader, rank + 1)
    load_part(part, w, dtype, DEV)
    load_part(reader, w_reader, dtype, DEV)
    x = rounded(torch.randn(180, 48, generator=torch.Generator().manual_seed(rank)), dtype)
    kept = plain.latent_of(x, w, "m.", m, 1e-6)
    want = plain.latent_attention(x, w, "m.", m, kept)
    want_reader = plain.latent_attention(x, w_reader, "n.", m_reader, kept)
    engine = PartEngine([part, reader], dtype, DEV, page, num_blocks=64, borrow={1: 0})
    whole = engine.run_cut("a", x, [180])
    check(whole[0], want, dtype)
    check(whole[1], want_reader, dtype)
    for sizes in ([1], [2], [9, 1, 1, 50], [128, 5]):
        cut = engine.run_cut("a", x, sizes)
        check(cut[0], want, dtype)
        check(cut[1], want_reader, dtype)
        if dtype == torch.float32:
            torch.testing.assert_close(cut[0], whole[0], rtol=2e-5, atol=2e-5)
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page", [(6, 4), (16, 16), (128, 8), (129, 16)])
def test_a_marked_latent_just_inside_and_just_outside_the_window(dtype, window, page):
    part, m = latent_part(2, 8, 4, 8, 16, window, scale=1.0)
    w = latent_weights(part, window, wide=0.3)
    gen = torch.Generator().manual_seed(window)
    length, marked = window + 30, 13
    x = rounded(torch.randn(length, 48, generator=gen) * 0.3, dtype)
    # the marked token turns its shared key part up; every query looks along it with a channel of its second rotated
    # pair, whose frequency is so low that the pair hardly turns over the sequence
    w["m.dkv"][16:, :] = 0.0
    w["m.dkv"][16 + 2, 7] = 30.0
    w["m.q"][:, 7] = 0.0
    x[:, 7] = 0.03125
    x[marked, 7] = 1.0
    w["m.q"][8 + 2, 7] = w["m.q"][12 + 8 + 2, 7] = 40.0
    part, m = latent_part(2, 8, 4, 8, 16, window, scale=1.0, base=1e8)
    load_part(part, w, dtype, DEV)
    kept = plain.latent_of(x, w, "m.", m, 1e-6)
    want = plain.latent_attention(x, w, "m.", m, kept)
    last_inside = marked + window - 1
    engine = PartEngine([part], dtype, DEV, page, num_blocks=64)
    for sizes in ([length], [last_inside, 1, 1, 1], [marked + 1, 1], [3, 2]):
        got = engine.run_cut("a", x, sizes)[0]
        check(got[marked:last_inside + 3], want[marked:last_inside + 3], dtype)
        check(got, want, dtype)
    # the oracle shows the edge: hiding the marked row changes the last token inside and not the next one
    hidden = (kept[0].clone(), kept[1].clone())
    hidden[1][marked] = 0.0
    blind = plain.latent_attention(x, w, "m.", m, hidden)
    assert float((want[last_inside] - blind[last_inside]).abs().max()) > 1e-3
    # (the next token's row is computed from rows that no longer hold the marked one, whatever it held)
    far = (kept[0].clone(), kept[1].clone())
    far[0][marked] = 0.0
    far[1][marked] = 0.0
    gone = plain.latent_attention(x, w, "m.", m, far)
    torch.testing.assert_close(want[last_inside + 1:], gone[last_inside + 1:], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_gate_reads_the_mixers_own_input(dtype):
    part, m = latent_part(2, 8, 4, 8, 16, None)
    w = latent_weights(part, 4)
    w["m.g"] = rounded(w["m.g"] * 10)
    load_part(part, w, dtype, DEV)
    x = rounded(torch.randn(12, 48, generator=torch.Generator().manual_seed(2)), dtype)
    want = plain.latent_attention(x, w, "m.", m, plain.latent_of(x, w, "m.", m, 1e-6))
    check(PartEngine([part], dtype, DEV, 8).run_cut("a", x, [12])[0], want, dtype)


# ------------------------------------------------------------------------------------------ which kernel runs
def test_which_sizes_take_the_matrix_core_kernels():
    def pages(kv, dim, vdim, page):
        return (torch.zeros(4, kv, page, dim, dtype=torch.bfloat16, device=DEV),
                torch.zeros(4, kv, vdim, page, dtype=torch.bfloat16, device=DEV))
    q = torch.zeros(2, 8 * 64, dtype=torch.bfloat16, device=DEV)
    assert ops.mixed_attention_mfma_supported(q, *pages(2, 64, 64, 16), 8)
    assert ops.mixed_attention_mfma_supported(q, *pages(8, 64, 128, 8), 8)
    assert not ops.mixed_attention_mfma_supported(q, *pages(2, 64, 24, 16), 8)       # value channels no multiple of 16
    assert not ops.mixed_attention_mfma_supported(q, *pages(2, 64, 64, 4), 8)        # pages shorter than 8 tokens
    assert not ops.mixed_attention_mfma_supported(q.float(), *pages(2, 64, 64, 16), 8)
    q = torch.zeros(2, 34 * 8, dtype=torch.bfloat16, device=DEV)
    assert not ops.mixed_attention_mfma_supported(q, *pages(2, 8, 16, 16), 34)       # 17 query heads a key/value head


@pytest.mark.parametrize("portions", [False, True])
@pytest.mark.parametrize("heads,kv,dim,vdim,window,cap", [(8, 2, 64, 32, 21, 15.0), (6, 2, 24, 32, None, None),
                                                          (5, 5, 128, 16, 100, 7.0), (16, 1, 32, 48, 3, None)])
def test_matrix_core_and_plain_attention_agree(portions, heads, kv, dim, vdim, window, cap):
    """The two kernels on the same pages, block table and queries: tokens of three requests side by side, one of them
    with a single token at a high position."""
    gen = torch.Generator().manual_seed(heads * dim)
    page, n_pages = 8, 40
    keys = (torch.randn(n_pages, kv, page, dim, generator=gen) * 0.5).to(torch.bfloat16).to(DEV)
    values = torch.randn(n_pages, kv, vdim, page, generator=gen).to(torch.bfloat16).to(DEV)
    table = torch.randperm(n_pages, generator=gen)[:36].view(3, 12).to(torch.int32).to(DEV)
    lengths = [(0, 37), (60, 9), (90, 1)]                        # (first position, tokens) of the three requests
    entry = torch.tensor(sum([[e] * n for e, (_, n) in enumerate(lengths)], []), dtype=torch.int32, device=DEV)
    position = torch.tensor(sum([list(range(p, p + n)) for p, n in lengths], []), dtype=torch.int32, device=DEV)
    q = torch.randn(entry.numel(), heads * dim, generator=gen).to(torch.bfloat16).to(DEV)
    talk = (torch.eye(heads) + 0.3 * torch.randn(heads, heads, generator=gen)).to(DEV)
    freq = (1.0 / (50.0 ** (torch.arange(0, vdim, 2, dtype=torch.float64) / vdim))).float().to(DEV)
    args = (q, keys, values, table, entry, position, heads, window or 0, dim ** -0.5, cap or 0.0, 1.0, talk, freq, "half")
    want = ops.mixed_attention_plain(*args)
    got = ops.mixed_attention_mfma(*args, portions=portions, max_context=91)
    check(got, want, torch.bfloat16)
    if not portions:
        # a token's keys dealt out to several workgroups (as a step of few tokens with long contexts has them)
        check(ops.mixed_attention_mfma(*args, portions=False, max_context=4096), want, torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_many_wide_heads_in_the_plain_kernel(dtype):
    """64 heads of 64 + 64 channels: more LDS than a workgroup gets unasked, and (in bfloat16) more query heads a
    key/value head than the matrix-core kernel has slots."""
    part, m = mixed_part(64, 2, 64, 64, 20, 10.0, 32)
    w = mixed_weights(part, 5)
    load_part(part, w, dtype, DEV)
    x = rounded(torch.randn(45, 48, generator=torch.Generator().manual_seed(3)), dtype)
    want = plain.attention(x, w, "m.", m)
    engine = PartEngine([part], dtype, DEV, 16, num_blocks=8)
    check(engine.run_cut("a", x, [30, 1, 14])[0], want, dtype)
