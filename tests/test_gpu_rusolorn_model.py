"""The Rusolorn decoder in the engine against the plain implementation, for every way of cutting the work."""

import pytest
import torch

import helpers
from helpers import make_engine, mixed_trace, peak_pages, run_portions, token_ids
from plain import rusolorn_plain as plain
from rusolorn_helpers import RUSOLORN, load_plain, write_rusolorn
from somi_inference_amd.engine import StepEntry

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]

# The float32 engine against the float32 plain implementation: sums in another order only, but this design divides
# every mixer's output and every recurrent head's by its own root mean square, which passes rounding on.
F32_TOL = dict(atol=2e-4, rtol=3e-4)
ROW_RMS_SHARE = 0.10          # bfloat16: a single row may be off by this share of its own size


CLOSE_CALL = 0.05             # a router's decision within this share of a tie may go the other way in bfloat16


def assert_close(got, want, dtype, what="", per_row=False, close_calls=()):
    """``close_calls``: rows whose token some router decides within CLOSE_CALL of a tie.  bfloat16 rounds the router's
    input, so such a token may take another expert, which is a jump and no rounding error: those rows are not held to
    the bfloat16 bounds (they are few, which the caller checks; float32 holds every row)."""
    if dtype != "float32" and len(close_calls):
        got = got.clone().float().cpu()
        rows = torch.tensor(sorted(close_calls), dtype=torch.long)
        assert bool(torch.isfinite(got[rows]).all())
        got[rows] = want.float().cpu()[rows]
    if dtype == "float32":
        torch.testing.assert_close(got.float().cpu(), want.float().cpu(), msg=lambda m: f"{what}: {m}", **F32_TOL)
        return
    if got.dim() == 2 and got.shape[0] >= 16:        # the tensor's bounds are for many rows together
        helpers.assert_close(got, want, dtype, what, per_row=False)
    assert got.shape == want.shape and bool(torch.isfinite(got.float()).all()), f"{what}: shape or values that are not finite"
    if per_row or got.shape[0] < 16:
        error, want = (got.float().cpu() - want.float().cpu()), want.float().cpu()
        share = error.pow(2).mean(dim=-1).sqrt() / want.pow(2).mean(dim=-1).sqrt()
        over = (share > ROW_RMS_SHARE).nonzero().flatten().tolist()
        assert not over, f"{what}: rows {over[:8]} are off by {[round(float(share[i]), 4) for i in over[:8]]} of their own size"


NAMES = list(RUSOLORN)
KINDS = {"free": False, "steady": True}      # the recurrent mixers' keys independent of their queries, or equal to them


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("rusolorn")
    return {(kind, name): write_rusolorn(name, str(root / f"{kind}_{name}"), steady)
            for kind, steady in KINDS.items() for name in NAMES}


@pytest.fixture(scope="module")
def oracle(folders):
    """Plain logits of (kind, name, tokens), computed once."""
    cache, models = {}, {}

    def both(kind, name, tokens):
        key = (kind, name, tuple(tokens))
        if key not in cache:
            if (kind, name) not in models:
                models[(kind, name)] = load_plain(folders[(kind, name)])
            config, weights = models[(kind, name)]
            margins = []
            logits = plain.forward(config, weights, list(tokens), margins=margins)
            least = torch.stack(margins).min(dim=0).values if margins else torch.full((len(tokens),), float("inf"))
            rows = (least < CLOSE_CALL).nonzero().flatten().tolist()
            assert len(rows) <= max(2, len(tokens) // 8), f"{len(rows)} of {len(tokens)} tokens are routed by a close call"
            cache[key] = (logits, rows)
        return cache[key]

    def get(kind, name, tokens):
        return both(kind, name, tokens)[0]
    get.close_calls = lambda kind, name, tokens: both(kind, name, tokens)[1]
    return get


def vocab_of(name):
    return RUSOLORN[name]["config"].vocab


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("kind", list(KINDS))
def test_whole_prompts_and_the_stream_after_every_layer(kind, name, dtype, folders, oracle):
    if dtype == "bfloat16" and kind == "free":
        pytest.skip("bfloat16 is held to a bound on models whose recurrent heads are steady at the first tokens")
    runner, _ = make_engine(folders[(kind, name)], dtype, RUSOLORN[name]["block_size"], 48, max_requests=2)
    for length, seed in ((1, 1), (2, 2), (9, 3), (33, 4), (64, 5), (131, 6)):
        tokens = token_ids(vocab_of(name), length, seed)
        got = run_portions(runner, f"r{length}", tokens, [length])
        assert_close(got, oracle(kind, name, tokens), dtype, f"{name} {kind} {dtype} whole prompt of {length}", per_row=True,
                     close_calls=oracle.close_calls(kind, name, tokens))
    runner.cache.check_invariants()
    assert runner.cache.free_pages() == [48] * len(runner.cache.groups)
    if dtype == "float32":
        # the residual stream after every layer, layer by layer
        config, weights = load_plain(folders[(kind, name)])
        tokens = token_ids(vocab_of(name), 40, 8)
        _, layers = plain.forward(config, weights, tokens, keep_layers=True)
        kept = []
        for layer in runner.model.layers:
            def forward(stream, step, cache, inner=layer.forward):
                inner(stream, step, cache)
                kept.append(stream.settle().clone().cpu())
            layer.forward = forward
        run_portions(runner, "layers", tokens, [40])
        for index, (got, want) in enumerate(zip(kept, layers)):
            torch.testing.assert_close(got, want, msg=lambda m: f"{name} after layer {index}: {m}", **F32_TOL)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_long_decoding_token_by_token(name, dtype, folders, oracle):
    """The decoded tokens pass every window and page edge of the configuration."""
    runner, _ = make_engine(folders[("steady", name)], dtype, RUSOLORN[name]["block_size"], 24, max_requests=2)
    for prefill, decoded in ((3, 90), (40, 120)):
        tokens = token_ids(vocab_of(name), prefill + decoded, 11 * prefill)
        got = run_portions(runner, "d", tokens, [prefill] + [1] * decoded)
        assert_close(got, oracle("steady", name, tokens), dtype, f"{name} {dtype} {prefill} + {decoded} decoded", per_row=True,
                     close_calls=oracle.close_calls("steady", name, tokens))
        if dtype == "float32":
            whole = run_portions(runner, "w", tokens, [prefill + decoded])
            assert torch.equal(got, whole), "float32 logits differ between decoding and the whole prompt"
    assert runner.graph_replays > 0          # decoded tokens took the captured step ...
    assert len(runner._graphs) <= 4          # ... which is captured once per shape, not once per step


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_several_sizes_down_to_two(name, dtype, folders, oracle):
    runner, _ = make_engine(folders[("steady", name)], dtype, RUSOLORN[name]["block_size"], 24, max_requests=2)
    tokens = token_ids(vocab_of(name), 170, 21)
    want = oracle("steady", name, tokens)
    whole = run_portions(runner, "w", tokens, [170])
    for sizes in ([2], [7, 2, 5, 3, 11], [16], [17, 15], [64, 2, 1, 1, 40], [1]):
        got = run_portions(runner, "p", tokens, sizes)
        assert_close(got, want, dtype, f"{name} {dtype} portions of {sizes}", per_row=True,
                     close_calls=oracle.close_calls("steady", name, tokens))
        if dtype == "float32":
            assert torch.equal(got, whole), f"float32 logits depend on the portions {sizes}"
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_requests_together_with_pages_and_slots_used_again(name, dtype, folders, oracle):
    """Up to four live requests (the slots there are), portions beside single tokens, in a pool that only holds what is
    live: every request's logits equal those it gets alone."""
    block = RUSOLORN[name]["block_size"]
    lengths = {"a": 95, "b": 1, "c": 33, "d": 140, "e": 2, "f": 64, "g": 77, "h": 18, "i": 120}
    requests = {rid: token_ids(vocab_of(name), n, 100 + n) for rid, n in lengths.items()}
    steps = mixed_trace(requests, seed=5, max_live=4)
    runner, _ = make_engine(folders[("steady", name)], dtype, block, peak_pages(steps, block), max_requests=4)
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
        assert_close(rows, oracle("steady", name, tokens), dtype, f"{name} {dtype} request {rid} in mixed batches", per_row=True,
                     close_calls=oracle.close_calls("steady", name, tokens))
        if dtype == "float32":
            assert torch.equal(rows, alone[rid]), f"float32 logits of request {rid} depend on the batch"
    assert runner.cache.free_pages() == [g.pool.num_pages for g in runner.cache.groups]


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_used_again_starts_from_zero(dtype, folders):
    runner, _ = make_engine(folders[("steady", "A")], dtype, 16, 16, max_requests=1)
    tokens = token_ids(vocab_of("A"), 40, 9)
    first = run_portions(runner, "one", tokens, [40])
    run_portions(runner, "other", token_ids(vocab_of("A"), 55, 10), [30, 25])
    again = run_portions(runner, "one", tokens, [13, 27])
    if dtype == "float32":
        assert torch.equal(first, again)
    else:
        assert_close(again, first, dtype, "the same request in a slot that was used in between")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_greedy_generation_through_the_entry_point(name, dtype, folders):
    from somi_inference_amd import LLM
    config, weights = load_plain(folders[("steady", name)])
    prompts = [token_ids(vocab_of(name), n, 60 + n) for n in (5, 23, 1, 48)]
    new_tokens = 12
    llm = LLM(folders[("steady", name)], dtype=dtype, num_blocks=32, block_size=RUSOLORN[name]["block_size"],
              max_concurrent=3, max_num_batched_tokens=32, eos_token_id=-1)
    got = llm.generate(prompts, max_new_tokens=new_tokens, temperature=0.0)
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == new_tokens
        sequence = list(prompt)
        for token in tokens:
            logits = plain.forward(config, weights, sequence)[-1]
            best = int(logits.argmax())
            if token != best:
                # a near tie may flip in bfloat16 (and, by a hair, in another order of float32 sums)
                gap = float(logits[best] - logits[token])
                assert gap < (1e-4 if dtype == "float32" else 0.05), f"token {token} instead of {best} (gap {gap})"
            sequence.append(token)
    llm.runner.cache.check_invariants()


def test_command_line_writes_a_random_model_and_generates_from_it(tmp_path):
    """The command line on a configuration file alone: seeded random weights into a folder, then greedy generation and
    sampling with a temperature, top-k and top-p from that folder."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    config_file, folder, out_file = tmp_path / "config.json", tmp_path / "model", tmp_path / "out.jsonl"
    config_file.write_text(json.dumps(RUSOLORN["D"]["config"].to_dict()))
    cli = [sys.executable, "-m", "somi_inference_amd.entrypoints.cli"]
    done = subprocess.run(cli + ["--write-random-model", str(folder), "--config-json", str(config_file), "--random-seed", "3"],
                          cwd=root, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    prompt = token_ids(vocab_of("D"), 9, 4)
    common = ["--model-name", str(folder), "--dtype", "float32", "--num-blocks", "8", "--max-new-tokens", "6",
              "--prompt-ids", ",".join(map(str, prompt)), "--output-file", str(out_file)]
    done = subprocess.run(cli + common + ["--temperature", "0.0"], cwd=root, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    record = json.loads(done.stdout.strip().splitlines()[-1])
    config, weights = load_plain(str(folder))
    sequence = list(prompt)
    for token in record["output"]:
        logits = plain.forward(config, weights, sequence)[-1]
        assert float(logits.max() - logits[token]) < 1e-4
        sequence.append(token)
    assert record["prompt"] == prompt and len(record["output"]) == 6
    done = subprocess.run(cli + common + ["--temperature", "0.9", "--top-k", "5", "--top-p", "0.9", "--seed", "7"],
                          cwd=root, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    sampled = json.loads(done.stdout.strip().splitlines()[-1])["output"]
    sequence = list(prompt)
    for token in sampled:                      # every sampled token is among the five most likely ones
        logits = plain.forward(config, weights, sequence)[-1]
        assert token in logits.topk(5).indices.tolist()
        sequence.append(token)


def test_a_preempted_request_is_recomputed_from_an_empty_state(folders):
    """A pool too small for three requests: one is preempted, gives back its pages and its state slot, and is run
    again from its first token later; its recurrent state and its convolution's inputs must start from zero again."""
    from somi_inference_amd import LLM
    folder = folders[("steady", "B")]                 # its windows never pass a page, so a request's pages only grow
    prompts = [token_ids(vocab_of("B"), n, 30 + n) for n in (30, 28, 25)]
    roomy = LLM(folder, dtype="float32", block_size=8, num_blocks=64, max_concurrent=3, eos_token_id=-1)
    want = roomy.generate(prompts, max_new_tokens=24, temperature=0.0)
    tight = LLM(folder, dtype="float32", block_size=8, num_blocks=14, max_concurrent=3, eos_token_id=-1)
    got = tight.generate(prompts, max_new_tokens=24, temperature=0.0)
    assert tight.scheduler.preemptions > 0 and roomy.scheduler.preemptions == 0
    assert got == want
    tight.kv_manager.check_invariants()
