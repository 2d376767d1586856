"""Random small Gizilorn configurations (layer orders with and without layers that read another's latent and see
further or less far than their lender, one to eight streams or none, query heads a key/value head that are no power
of two, key and value sizes that are and are not what the matrix-core kernels take, fewer rotated channels than a head
has, windows from one key to none, caps or none, layers without a feed-forward, widths that are no multiple of 8, page
sizes) under random mixed traces with so few pages that they are used again: the engine against the plain
implementation and against itself on the whole prompt."""

import random

import pytest
import torch

from gizilorn_helpers import GIZILORN, attention, latent, load_plain, write_gizilorn
from helpers import make_engine, mixed_trace, peak_pages, token_ids
from plain import gizilorn_plain as plain
from somi_inference_amd.config import GizilornConfig, GizilornDense
from somi_inference_amd.engine import StepEntry
from test_gpu_gizilorn_model import assert_close

pytestmark = pytest.mark.gpu


def random_config(rng: random.Random) -> GizilornConfig:
    def mlp():
        return None if rng.random() < 0.25 else GizilornDense(rng.choice([8, 20, 36, 64, 96]))

    def window():
        return rng.choice([None, 1, 2, 5, 16, 17, 33, 64, 70, 129])

    layers, lenders = [], []
    for index in range(rng.choice([1, 2, 3, 4, 5])):
        if rng.random() < 0.5:
            if lenders and rng.random() < 0.5:
                source = rng.choice(lenders)
                m = layers[source].mixer
                layers.append(latent(rng.choice([1, 2, 5, 18]), rng.choice([8, 16, 24]), m.rot_dim, rng.choice([8, 16, 20]),
                                     m.kv_rank, window(), base=m.rot_base, scale=rng.choice([0.1, 0.3]), kv_from=source,
                                     mlp=mlp()))
                continue
            layers.append(latent(rng.choice([1, 2, 3, 6, 17, 20]), rng.choice([8, 12, 16, 32]), rng.choice([2, 4, 8, 16, 32]),
                                 rng.choice([8, 16, 24]), rng.choice([16, 24, 32, 48, 64, 96, 160]), window(),
                                 base=rng.choice([10.0, 1000.0, 100000.0]), scale=rng.choice([0.1, 0.2, 0.4]), mlp=mlp()))
            lenders.append(index)
        else:
            kv = rng.choice([1, 2, 3, 4])
            dim = rng.choice([8, 12, 16, 24, 32, 64])
            layers.append(attention(kv * rng.choice([1, 2, 3, 4, 6]), kv, dim, rng.choice([2, 8, 16, 24, 32, 48, 64]), window(),
                                    rng.choice([None, 5.0, 25.0, 50.0]), rng.choice([d for d in (2, 4, 8, 12, 16, 32, 64) if d <= dim]),
                                    base=rng.choice([10.0, 1000.0, 50000.0]), scale=rng.choice([0.1, 0.2, 0.4]), mlp=mlp()))
    return GizilornConfig(vocab=rng.choice([61, 97, 130, 256, 301]), width=rng.choice([40, 44, 64, 72, 100, 132]),
                          norm_eps=rng.choice([1e-6, 1e-5]), streams=rng.choice([None, 1, 2, 3, 4, 8]), layers=tuple(layers))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(24))
def test_random_configuration_under_a_random_mixed_trace(seed, dtype, tmp_path):
    rng = random.Random(seed)
    config = random_config(rng)
    block_size = rng.choice([4, 8, 16, 32])
    GIZILORN["random"] = dict(block_size=block_size, seed=rng.randrange(1000), config=config)
    try:
        folder = write_gizilorn("random", str(tmp_path / "model"), peaky=rng.random() < 0.5)
    finally:
        del GIZILORN["random"]
    weights, plain_config = load_plain(folder)
    lengths = {f"r{i}": rng.choice([1, 2, 3, 17, 33, 45, 64, 70, 100, 150]) for i in range(rng.randrange(3, 7))}
    requests = {rid: token_ids(config.vocab, n, rng.randrange(10000)) for rid, n in lengths.items()}
    sizes = tuple(rng.choice([1, 2, 3, 5, 7, 8, 9, 11, 16, 17, 31, 64, 65]) for _ in range(6))
    steps = mixed_trace(requests, seed=rng.randrange(1000), portion_sizes=sizes)
    pages = peak_pages(steps, block_size)
    runner, _ = make_engine(folder, dtype, block_size, pages, max_requests=4)
    rows = {rid: [] for rid in requests}
    for entries, ends in steps:
        batch = []
        for rid, start, count in entries:
            if not runner.cache.has(rid):
                runner.begin(rid)
            batch.append(StepEntry(rid, requests[rid][start:start + count], list(range(count))))
        logits = runner.step(batch).cpu()
        at = 0
        for rid, start, count in entries:
            rows[rid].append(logits[at:at + count])
            at += count
        for rid in ends:
            runner.end(rid)
        runner.cache.check_invariants()
    what = f"seed {seed} {dtype} {config.to_dict()} pages of {block_size}"
    for rid, tokens in requests.items():
        mixed = torch.cat(rows[rid])
        want = plain.forward(plain_config, weights, tokens, dtype=torch.float32)[0]
        assert_close(mixed, want, dtype, f"{what}: request {rid} of {lengths[rid]} in a mixed trace")
        runner.begin("whole")
        whole = runner.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
        runner.end("whole")
        if dtype == "float32":
            torch.testing.assert_close(mixed, whole, atol=2e-5, rtol=2e-5, msg=lambda m: f"{what}: logits of {rid} depend on the cutting: {m}")
        else:
            assert_close(mixed, whole, dtype, f"{what}: request {rid} against its whole prompt")
    assert runner.cache.free_pages() == [g.pool.num_pages for g in runner.cache.groups]
