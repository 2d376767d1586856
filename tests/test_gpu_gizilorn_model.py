"""The Gizilorn decoder in the engine against the plain implementation, for every way of cutting the work."""

import json
import os
import subprocess
import sys

import pytest
import torch

from gizilorn_helpers import GIZILORN, load_plain, write_gizilorn
from helpers import make_engine, mixed_trace, peak_pages, run_portions, token_ids
from plain import gizilorn_plain as plain
from somi_inference_amd.engine import StepEntry

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
# The float32 engine against the float32 plain implementation: sums in another order only.
F32_TOL = dict(atol=3e-4, rtol=3e-4)
# bfloat16: a single row may be off by this share of its own size; a row from a wrong key, window edge, page or
# neighbour is off by about its own size
ROW_RMS_SHARE = 0.12
NAMES = list(GIZILORN)
KINDS = {"plain": False, "peaky": True}


def assert_close(got, want, dtype, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape and bool(torch.isfinite(got).all()), f"{what}: shape or values that are not finite"
    if dtype == "float32":
        torch.testing.assert_close(got, want, msg=lambda m: f"{what}: {m}", **F32_TOL)
        return
    share = (got - want).pow(2).mean(dim=-1).sqrt() / want.pow(2).mean(dim=-1).sqrt()
    over = (share > ROW_RMS_SHARE).nonzero().flatten().tolist()
    assert not over, f"{what}: rows {over[:8]} are off by {[round(float(share[i]), 4) for i in over[:8]]} of their own size"
    assert float(share.median()) < ROW_RMS_SHARE / 3, f"{what}: the rows' median error is {float(share.median()):.4f} of their size"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("gizilorn")
    return {(kind, name): write_gizilorn(name, str(root / f"{kind}_{name}"), peaky)
            for kind, peaky in KINDS.items() for name in NAMES}


@pytest.fixture(scope="module")
def oracle(folders):
    """Plain logits of (kind, name, tokens), computed once."""
    cache, models = {}, {}

    def get(kind, name, tokens):
        key = (kind, name, tuple(tokens))
        if key not in cache:
            if (kind, name) not in models:
                models[(kind, name)] = load_plain(folders[(kind, name)])
            weights, config = models[(kind, name)]
            cache[key] = plain.forward(config, weights, list(tokens), dtype=torch.float32)[0]
        return cache[key]
    return get


def vocab_of(name):
    return GIZILORN[name]["config"].vocab


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("kind", list(KINDS))
def test_whole_prompts_and_the_streams_sum_after_every_layer(kind, name, dtype, folders, oracle):
    runner, _ = make_engine(folders[(kind, name)], dtype, GIZILORN[name]["block_size"], 48, max_requests=2)
    for length, seed in ((1, 1), (2, 2), (9, 3), (33, 4), (64, 5), (150, 6)):
        tokens = token_ids(vocab_of(name), length, seed)
        got = run_portions(runner, f"r{length}", tokens, [length])
        assert_close(got, oracle(kind, name, tokens), dtype, f"{name} {kind} {dtype} whole prompt of {length}")
    runner.cache.check_invariants()
    assert runner.cache.free_pages() == [48] * len(runner.cache.groups)
    if dtype == "float32":
        weights, config = load_plain(folders[(kind, name)])
        tokens = token_ids(vocab_of(name), 40, 8)
        _, layers = plain.forward(config, weights, tokens, dtype=torch.float32)
        kept = []
        for layer in runner.model.layers:
            def forward(stream, step, cache, inner=layer.forward):
                inner(stream, step, cache)
                kept.append(stream.settle().clone().cpu())
            layer.forward = forward
        run_portions(runner, "layers", tokens, [40])
        assert len(kept) == len(layers)
        for index, (got, want) in enumerate(zip(kept, layers)):
            torch.testing.assert_close(got, want, msg=lambda m: f"{name} after layer {index}: {m}", **F32_TOL)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_long_decoding_token_by_token(name, dtype, folders, oracle):
    """The decoded tokens pass many page edges and every window; the first tokens of a sequence are decoded one by
    one as well."""
    runner, _ = make_engine(folders[("peaky", name)], dtype, GIZILORN[name]["block_size"], 64, max_requests=2)
    for prefill, decoded in ((1, 70), (40, 170)):
        tokens = token_ids(vocab_of(name), prefill + decoded, 11 * prefill)
        got = run_portions(runner, "d", tokens, [prefill] + [1] * decoded)
        assert_close(got, oracle("peaky", name, tokens), dtype, f"{name} {dtype} {prefill} + {decoded} decoded")
        whole = run_portions(runner, "w", tokens, [prefill + decoded])
        if dtype == "float32":
            torch.testing.assert_close(got, whole, atol=2e-5, rtol=2e-5)
        else:
            assert_close(got, whole, dtype, f"{name} decoding against the whole prompt")
    assert runner.graph_replays > 0          # decoded tokens took the captured step ...
    assert len(runner._graphs) <= 4          # ... which is captured once per shape, not once per step


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_several_sizes_down_to_two(name, dtype, folders, oracle):
    runner, _ = make_engine(folders[("peaky", name)], dtype, GIZILORN[name]["block_size"], 64, max_requests=2)
    tokens = token_ids(vocab_of(name), 170, 21)
    want = oracle("peaky", name, tokens)
    whole = run_portions(runner, "w", tokens, [170])
    for sizes in ([2], [7, 2, 5, 3, 11], [16], [17, 15], [64, 2, 1, 1, 40], [1]):
        got = run_portions(runner, "p", tokens, sizes)
        assert_close(got, want, dtype, f"{name} {dtype} portions of {sizes}")
        if dtype == "float32":
            torch.testing.assert_close(got, whole, atol=2e-5, rtol=2e-5, msg=lambda m: f"float32 logits depend on the portions {sizes}: {m}")
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_requests_together_with_pages_and_slots_used_again(name, dtype, folders, oracle):
    """Up to four live requests (the slots there are), portions beside single tokens, in a pool that only holds what is
    live: every request's logits equal those it gets alone."""
    block = GIZILORN[name]["block_size"]
    lengths = {"a": 95, "b": 1, "c": 33, "d": 140, "e": 2, "f": 64, "g": 77, "h": 18, "i": 120}
    requests = {rid: token_ids(vocab_of(name), n, 100 + n) for rid, n in lengths.items()}
    steps = mixed_trace(requests, seed=5, max_live=4)
    runner, _ = make_engine(folders[("peaky", name)], dtype, block, peak_pages(steps, block), max_requests=4)
    alone = {rid: run_portions(runner, "alone", tokens, [len(tokens)]) for rid, tokens in requests.items()}
    got = {rid: [] for rid in requests}
    slots_seen = set()
    for entries, ends in steps:
        batch = []
        for rid, start, count in entries:
            if not runner.cache.has(rid):
                runner.begin(rid)
                slots_seen.add(runner.cache.state_slot(rid))
            batch.append(StepEntry(rid, requests[rid][start:start + count], list(range(count))))
        logits = runner.step(batch).cpu()
        at = 0
        for rid, _, count in entries:
            got[rid].append(logits[at:at + count].clone())
            at += count
        for rid in ends:
            runner.end(rid)
        runner.cache.check_invariants()
    assert len(slots_seen) <= 4 < len(requests)               # slots were used again
    for rid, tokens in requests.items():
        rows = torch.cat(got[rid])
        assert_close(rows, oracle("peaky", name, tokens), dtype, f"{name} {dtype} request {rid} in mixed batches")
        if dtype == "float32":
            torch.testing.assert_close(rows, alone[rid], atol=2e-5, rtol=2e-5,
                                       msg=lambda m: f"float32 logits of request {rid} depend on the batch: {m}")
    assert runner.cache.free_pages() == [g.pool.num_pages for g in runner.cache.groups]


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_a_window_gave_back_are_not_missed(dtype, folders, oracle):
    """A pool far smaller than the sequence: every layer has a window (or reads a cache kept for its reader's), so
    pages behind it return to the pool while the request is live and are handed out again to the same request."""
    name = "C"
    runner, _ = make_engine(folders[("peaky", name)], dtype, 4, 12, max_requests=1)
    tokens = token_ids(vocab_of(name), 260, 31)
    got = run_portions(runner, "long", tokens, [20, 1, 1, 9, 2])
    assert_close(got, oracle("peaky", name, tokens), dtype, f"{name} {dtype} in a pool of 48 tokens")
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_greedy_generation_through_the_entry_point(name, dtype, folders):
    from somi_inference_amd import LLM
    weights, config = load_plain(folders[("plain", name)])
    prompts = [token_ids(vocab_of(name), n, 60 + n) for n in (5, 23, 1, 48)]
    new_tokens = 12
    llm = LLM(folders[("plain", name)], dtype=dtype, num_blocks=48, block_size=GIZILORN[name]["block_size"],
              max_concurrent=3, max_num_batched_tokens=32, eos_token_id=-1)
    got = llm.generate(prompts, max_new_tokens=new_tokens, temperature=0.0)
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == new_tokens
        sequence = list(prompt)
        for token in tokens:
            logits = plain.forward(config, weights, sequence, dtype=torch.float32)[0][-1]
            best = int(logits.argmax())
            if token != best:
                # a near tie may flip in bfloat16 (and, by a hair, in another order of float32 sums)
                gap = float(logits[best] - logits[token]) / float(logits.std())
                assert gap < (1e-4 if dtype == "float32" else 0.08), f"token {token} instead of {best} (gap {gap})"
            sequence.append(token)
    llm.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_of_a_trace_as_a_subprocess(dtype, folders, tmp_path, oracle):
    """bin/trace_run on a model folder: a mixed trace with four slots and a pool that only holds what is live."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    name = "A"
    requests = {rid: token_ids(vocab_of(name), n, 200 + n) for rid, n in {"a": 70, "b": 3, "c": 41, "d": 90, "e": 25, "f": 1}.items()}
    steps = mixed_trace(requests, seed=9, max_live=4)
    lines = []
    for index, (entries, ends) in enumerate(steps):
        lines.append(json.dumps({"step": index, "end": ends, "entries": [
            {"id": rid, "tokens": requests[rid][start:start + count], "want": list(range(count))} for rid, start, count in entries]}))
    out = tmp_path / "out"
    done = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folders[("plain", name)],
                           "--dtype", dtype, "--out", str(out), "--max-tokens", str(peak_pages(steps, 64) * 64)],
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600, cwd=root)
    assert done.returncode == 0, done.stderr[-3000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    got = {rid: [] for rid in requests}
    import numpy as np
    for index, (entries, _) in enumerate(steps):
        rows = torch.from_numpy(np.fromfile(out / f"{index}.f32", dtype="<f4").reshape(-1, vocab_of(name)).copy())
        at = 0
        for rid, _, count in entries:
            got[rid].append(rows[at:at + count])
            at += count
    for rid, tokens in requests.items():
        assert_close(torch.cat(got[rid]), oracle("plain", name, tokens), dtype, f"replayed request {rid}")
