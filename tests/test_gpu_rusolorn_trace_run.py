"""bin/trace_run on a Rusolorn model folder as a user runs it: a subprocess fed JSON lines; whole prompts, decoding, portions
and a mixed trace in a pool that only holds what is live, with four request slots that are used again."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import mixed_trace, token_ids
from rusolorn_helpers import RUSOLORN, load_plain, write_rusolorn
from plain import rusolorn_plain as plain
from test_gpu_rusolorn_model import CLOSE_CALL, assert_close

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_trace(folder, dtype, out_dir, max_tokens, steps):
    lines = "".join(json.dumps(s) + "\n" for s in steps)
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out_dir), "--max-tokens", str(max_tokens)],
                          input=lines, capture_output=True, text=True, timeout=600, cwd="/")
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]


def read_logits(out_dir, step, vocab):
    data = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
    assert data.size % vocab == 0
    return torch.from_numpy(data.reshape(-1, vocab).copy())


def round64(n):
    return (n + 63) // 64 * 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_of_a_rusolorn_folder(dtype, tmp_path):
    name = "A"
    folder = write_rusolorn(name, str(tmp_path / "model"), steady=True)
    vocab = RUSOLORN[name]["config"].vocab
    config, weights = load_plain(folder)
    requests = {rid: token_ids(vocab, n, 70 + i) for i, (rid, n) in
                enumerate({"a": 70, "b": 45, "c": 100, "d": 33, "e": 130, "f": 1}.items())}
    want, close = {}, {}
    for rid, tokens in requests.items():
        margins = []
        want[rid] = plain.forward(config, weights, tokens, margins=margins)
        close[rid] = set((torch.stack(margins).min(dim=0).values < CLOSE_CALL).nonzero().flatten().tolist())

    # most of a request in one step, its last 40 tokens one by one (they pass the windows of 24 and 36 tokens)
    b = requests["e"]
    steps, expect = [{"step": 0, "entries": [{"id": "dec", "tokens": b[:-40], "want": [0, len(b) - 41]}], "end": []}], {}
    expect[0] = want["e"][[0, len(b) - 41]]
    skip = {0: [i for i, place in enumerate((0, len(b) - 41)) if place in close["e"]]}
    for number, i in enumerate(range(len(b) - 40, len(b)), start=1):
        steps.append({"step": number, "entries": [{"id": "dec", "tokens": [b[i]], "want": [0]}],
                      "end": ["dec"] if i == len(b) - 1 else []})
        expect[number] = want["e"][i:i + 1]
        skip[number] = [0] if i in close["e"] else []
    out1 = tmp_path / "decode"
    run_trace(folder, dtype, out1, round64(len(b)), steps)
    for step, logits in expect.items():
        assert_close(read_logits(out1, step, vocab), logits, dtype, f"{dtype} step {step}", per_row=True, close_calls=skip[step])

    # mixed: up to four live requests, portions beside single tokens, the pool sized by what is live at once
    trace = mixed_trace(requests, seed=3)
    live, peak = {}, 0
    for entries, ends in trace:
        for rid, start, count in entries:
            live[rid] = len(requests[rid])
        peak = max(peak, sum(round64(n) for n in live.values()))
        for rid in ends:
            del live[rid]
    assert peak < sum(round64(len(t)) for t in requests.values())
    steps, expect, skip = [], {}, {}
    for number, (entries, ends) in enumerate(trace):
        items, rows, at = [], [], 0
        for rid, start, count in entries:
            wanted = [] if (number + start) % 5 == 0 and count > 1 else list(range(count))
            items.append({"id": rid, "tokens": requests[rid][start:start + count], "want": wanted})
            rows.append(want[rid][[start + w for w in wanted]])
            skip.setdefault(number, []).extend(at + i for i, w in enumerate(wanted) if start + w in close[rid])
            at += len(wanted)
        steps.append({"step": number, "entries": items, "end": ends})
        if sum(r.shape[0] for r in rows):
            expect[number] = torch.cat(rows)
    out2 = tmp_path / "mixed"
    run_trace(folder, dtype, out2, peak, steps)
    for step, logits in expect.items():
        assert_close(read_logits(out2, step, vocab), logits, dtype, f"{dtype} mixed step {step}", per_row=True,
                     close_calls=skip.get(step, []))
    assert sorted(int(f[:-4]) for f in os.listdir(out2) if f.endswith(".f32")) == sorted(expect)
