"""Traces in the replay tool's format, the ways of running them, and the comparison with the
plain implementation."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def random_tokens(vocab, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def whole(requests):
    """Each request alone and whole, one after the other."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def last_decoded(requests, tail=32):
    """Most of each request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, seed=0, sizes=(2, 3, 5, 7, 16, 17, 24, 2, 31, 1)):
    """Each request alone, in portions of changing size, down to two tokens."""
    rng = random.Random(seed)
    steps = []
    for rid, toks in requests.items():
        i = 0
        k = rng.randrange(len(sizes))
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + n],
                                                          "want": list(range(n))}], "end": []})
            i += n
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests, max_live=4, seed=0, decode_tail=12, max_portion=24):
    """Up to ``max_live`` requests at a time: portions of some beside single decoded tokens of others;
    a request that ends makes room for the next, so its pages are used again.  Now and then a live
    request sits a step out."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}     # rid -> [tokens, fed]
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
            if rng.random() < 0.5:
                break     # stagger the starts
        entries, end = [], []
        for rid, (toks, fed) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.15:
                continue
            left = len(toks) - fed
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.randint(2, max_portion), left - decode_tail) if left - decode_tail >= 2 else left - decode_tail
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": list(range(n))})
            live[rid][1] = fed + n
            if fed + n == len(toks):
                end.append(rid)
                del live[rid]
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def few_wanted(steps, seed=0, none=0.15):
    """The same steps with the logits of at most the last token of each entry wanted, and of some entries none:
    which rows a step wants then changes from step to step among steps of the same entries."""
    rng = random.Random(seed)
    out = []
    for st in steps:
        entries = [dict(e, want=[] if rng.random() < none else [len(e["tokens"]) - 1]) for e in st["entries"]]
        out.append(dict(st, entries=entries))
    return out


def random_wanted(steps, seed=0):
    """The same steps with wanted places drawn at random for every entry (all of them, the last one, none, or a
    few in any order, a place perhaps twice) and the entries of a step in a random order."""
    rng = random.Random(seed)
    out = []
    for st in steps:
        entries = []
        for e in st["entries"]:
            n, c = len(e["tokens"]), rng.random()
            want = list(range(n)) if c < 0.25 else [n - 1] if c < 0.6 else [] if c < 0.75 else \
                [rng.randrange(n) for _ in range(rng.randint(1, 4))]
            entries.append(dict(e, want=want))
        rng.shuffle(entries)
        out.append(dict(st, entries=entries))
    return out


def max_live_tokens(steps, round_to=64):
    """The largest sum over live requests of their token counts rounded up, at any step."""
    held, best = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        best = max(best, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return best


def run_in_process(engine, steps):
    """Drive Engine.step directly; returns {step: float32 array [wanted, vocab]}."""
    from zedinfer_amd.engine import StepEntry
    live, out = {}, {}
    for st in steps:
        entries = []
        for e in st["entries"]:
            if e["id"] not in live:
                live[e["id"]] = engine.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        lg = engine.step(entries)
        if lg is not None:
            out[st["step"]] = lg.cpu().numpy()
        for rid in st["end"]:
            engine.close(live.pop(rid))
        engine.cache.check()
    assert not engine.cache.live
    return out


def run_tool(model_dir, dtype, steps, out_dir, max_tokens, timeout=600, options=(), geometry=None, stderr_to=None):
    """Drive bin/trace_run as a child process, one step at a time, waiting for each 'done'.  ``options``
    are further command-line options, ``geometry`` a dict sent as the trace's geometry line;
    ``stderr_to`` is a file path that receives what the tool says on standard error."""
    os.makedirs(out_dir, exist_ok=True)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)] + [str(o) for o in options]
    err = open(stderr_to, "w") if stderr_to else None
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=err, text=True)
    try:
        if geometry is not None:
            p.stdin.write(json.dumps({"geometry": geometry}) + "\n")
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            line = p.stdout.readline().strip()
            assert line == f"done {st['step']}", f"expected 'done {st['step']}', got {line!r}"
        p.stdin.close()
        assert p.wait(timeout=timeout) == 0
    finally:
        if p.poll() is None:
            p.kill()
        if err:
            err.close()
    out = {}
    for st in steps:
        n = sum(len(e["want"]) for e in st["entries"])
        f = os.path.join(out_dir, f"{st['step']}.f32")
        if n:
            a = np.fromfile(f, dtype="<f4")
            out[st["step"]] = a.reshape(n, -1)
        else:
            assert not os.path.exists(f)
    return out


def compare(steps, outputs, reference, requests):
    """Match every written row with the plain implementation's logits at (request, position).
    Returns (largest absolute difference, mean absolute difference, largest |reference|, rows)."""
    fed = {}
    worst, total, count, scale = 0.0, 0.0, 0, 0.0
    first_bad = None
    for st in steps:
        row = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for w in e["want"]:
                got = outputs[st["step"]][row]
                ref = reference[e["id"]][base + w].numpy()
                d = np.abs(got - ref)
                if d.max() > worst:
                    worst = float(d.max())
                    first_bad = (st["step"], e["id"], base + w)
                total += float(d.mean())
                scale = max(scale, float(np.abs(ref).max()))
                count += 1
                row += 1
            fed[e["id"]] = base + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    return worst, total / max(count, 1), scale, count, first_bad
