"""Trace replay: the replayer on the CPU with the twins, and the bin/trace_run program on the GPU."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import TINIES, TOLERANCE, plain_logits, random_tokens, rel_err, write_tiny_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def make_trace(vocab, lengths=(70, 45, 90, 33, 64)):
    """Five requests, up to four live: portions of changing size (down to two tokens) beside single tokens,
    requests left out of some steps, everything wanted.  Returns (steps, prompts, most tokens held at once)."""
    prompts = {f"r{i}": random_tokens(vocab, n, seed=200 + i) for i, n in enumerate(lengths)}
    plans = {}
    for i, (r, toks) in enumerate(prompts.items()):
        body, tail = toks[:-5], toks[-5:]
        sizes, parts, k, j = [13 + i, 2, 7, 31], [], 0, 0
        while k < len(body):
            n = min(sizes[j % 4], len(body) - k)
            parts.append(body[k:k + n]); k += n; j += 1
        plans[r] = parts + [[t] for t in tail]
    waiting, live, steps, held, most = list(prompts), [], [], {}, 0
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in list(live):
            if (len(steps) + int(r[1:])) % 4 == 3 and len(live) > 1:
                continue
            part = plans[r].pop(0)
            entries.append({"id": r, "tokens": part, "want": list(range(len(part)))})
            held[r] = held.get(r, 0) + len(part)
            if not plans[r]:
                end.append(r)
                live.remove(r)
        most = max(most, sum(-(-n // 64) * 64 for n in held.values()))
        for r in end:
            del held[r]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps, prompts, most


def collect(steps, read):
    got = {}
    fed = {}
    for st in steps:
        rows = read(st)
        i = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for w in e["want"]:
                got.setdefault(e["id"], {})[base + w] = rows[i]
                i += 1
            fed[e["id"]] = base + len(e["tokens"])
    return got


def check(got, prompts, folder, tol):
    for r, toks in prompts.items():
        ref = plain_logits(folder, toks)
        mine = torch.stack([torch.as_tensor(got[r][p]) for p in range(len(toks))])
        assert rel_err(mine, ref) <= tol, r


@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_replayer_on_cpu(tmp_path, name):
    from simple_inference_amd.replay import TraceReplayer
    from twins import TwinKernels
    tiny = TINIES[name]
    folder = write_tiny_model(tmp_path, tiny, seed=31)
    steps, prompts, most = make_trace(tiny.config["vocab_size"])
    rp = TraceReplayer(folder, "float32", most, block_size=16, device="cpu", kernels=TwinKernels())
    got = collect(steps, lambda st: rp.step(st["entries"], st["end"]).numpy())
    check(got, prompts, folder, TOLERANCE["twins"])
    assert rp.cache.free_pages() == -(-most // 16) and not rp.ids


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["b", "c"])
def test_trace_run_program(tmp_path, name, dtype):
    tiny = TINIES[name]
    folder = write_tiny_model(tmp_path / "model", tiny, seed=32)
    steps, prompts, most = make_trace(tiny.config["vocab_size"])
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(most)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:                       # the next step is sent only after "done <step>"
        proc.stdin.write(json.dumps(st) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {st['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    vocab = tiny.config["vocab_size"]

    def read(st):
        wanted = sum(len(e["want"]) for e in st["entries"])
        arr = np.fromfile(out / f"{st['step']}.f32", dtype="<f4")
        assert arr.size == wanted * vocab
        return arr.reshape(wanted, vocab)
    got = collect(steps, read)
    check(got, prompts, folder, TOLERANCE["hip-f32" if dtype == "float32" else "hip-bf16"])
