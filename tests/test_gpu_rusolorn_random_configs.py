"""Random small Rusolorn configurations (head counts and groups, head sizes that are and are not multiples of 16,
widths that are no multiple of 8, windows from one token to longer than any request, taps, experts with and without
groups and a shared expert, layers with and without a feed-forward, page sizes) under random mixed traces with so few
pages that they are used again: the float32 engine against the plain implementation, and against itself whole."""

import random

import pytest
import torch

from helpers import make_engine, mixed_trace, peak_pages, token_ids
from plain import rusolorn_plain as plain
from rusolorn_helpers import RUSOLORN, layer, load_plain, write_rusolorn
from somi_inference_amd.config import RusolornConfig
from somi_inference_amd.engine import StepEntry
from test_gpu_rusolorn_model import CLOSE_CALL, assert_close

pytestmark = pytest.mark.gpu


def random_config(rng: random.Random) -> RusolornConfig:
    def mixer():
        groups = rng.choice([1, 2, 3])
        heads = groups * rng.choice([1, 2, 4])
        r_groups = rng.choice([1, 2])
        left = (heads, groups, rng.choice([8, 12, 16, 24, 32, 48, 64, 128]), rng.choice([1, 2, 5, 16, 17, 33, 64, 500]),
                rng.choice([0.1, 0.3, 0.6]))
        right = (r_groups * rng.choice([1, 2, 3]), r_groups, rng.choice([6, 8, 16, 20, 32, 64, 100]),
                 rng.choice([4, 8, 16, 24, 40, 64]), rng.choice([1, 2, 3, 4, 5]))
        return left, right

    def experts():
        if rng.random() < 0.2:
            return None
        groups = rng.choice([1, 1, 2, 3, 4])
        count = groups * rng.choice([1, 2, 3])
        keep = rng.randrange(1, groups + 1)
        out = dict(experts=count, top=rng.randrange(1, keep * (count // groups) + 1), ff=rng.choice([8, 12, 24, 40, 64]),
                   limit=rng.choice([0.5, 1.5, 7.0]), groups=groups, keep=keep)
        if rng.random() < 0.6:
            out.update(shared_ff=rng.choice([8, 20, 48]), shared_limit=rng.choice([1.0, 3.0]))
        return out
    layers = tuple(layer(*mixer(), experts()) for _ in range(rng.choice([1, 2, 3])))
    return RusolornConfig(vocab=rng.choice([61, 97, 130, 256, 301]), width=rng.choice([40, 44, 64, 72, 100, 136]),
                          norm_eps=rng.choice([1e-6, 1e-5]), embedding_scale=rng.choice([1.0, 3.0, 11.0]),
                          residual_mult=rng.choice([0.4, 1.0, 1.6]), token_side_dim=rng.choice([None, 3, 8, 16]),
                          layers=layers)


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration_under_a_random_mixed_trace(seed, tmp_path):
    rng = random.Random(seed)
    config = random_config(rng)
    block_size = rng.choice([4, 8, 16, 32])
    RUSOLORN["random"] = dict(block_size=block_size, seed=rng.randrange(1000), config=config)
    try:
        folder = write_rusolorn("random", str(tmp_path / "model"), steady=rng.random() < 0.5)
    finally:
        del RUSOLORN["random"]
    plain_config, weights = load_plain(folder)
    lengths = {f"r{i}": rng.choice([1, 2, 3, 17, 33, 45, 64, 70, 100, 129]) for i in range(rng.randrange(3, 7))}
    requests = {rid: token_ids(config.vocab, n, rng.randrange(10000)) for rid, n in lengths.items()}
    sizes = tuple(rng.choice([1, 2, 3, 5, 7, 8, 9, 11, 16, 17, 31, 64, 65]) for _ in range(6))
    steps = mixed_trace(requests, seed=rng.randrange(1000), portion_sizes=sizes)
    pages = peak_pages(steps, block_size)
    runner, _ = make_engine(folder, "float32", block_size, pages, max_requests=4)
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
    what = f"seed {seed} {config.to_dict()} pages of {block_size}"
    for rid, tokens in requests.items():
        mixed = torch.cat(rows[rid])
        margins = []
        want = plain.forward(plain_config, weights, tokens, margins=margins)
        # the plain implementation adds in another order: a router's tie within 1e-4 may go either way there too
        close = (torch.stack(margins).min(dim=0).values < 1e-4).nonzero().flatten().tolist() if margins else []
        keep = [i for i in range(len(tokens)) if i not in close]
        assert_close(mixed[keep], want[keep], "float32", f"{what}: request {rid} of {lengths[rid]} in a mixed trace")
        runner.begin("whole")
        whole = runner.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
        runner.end("whole")
        assert torch.equal(mixed, whole), f"{what}: float32 logits of {rid} depend on the cutting"
    assert runner.cache.free_pages() == [g.pool.num_pages for g in runner.cache.groups]
