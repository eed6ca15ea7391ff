"""Trace schedules for the replay tests: the same requests cut in different ways.

A request is a full token sequence (prompt + given "decoded" tokens).  Every schedule
asks for the logits at every position, so each can be compared row by row with the
plain implementation's whole-sequence logits.
"""
import io
import json
import os

import numpy as np


def whole(reqs):
    """Each request alone and whole: one step each."""
    steps = []
    for i, (rid, toks) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_one_by_one(reqs, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps, s = [], 0
    for rid, toks in reqs.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
            s += 1
        for i in range(head, len(toks)):
            steps.append({"step": s, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
            s += 1
    return steps


def portions(reqs, sizes=(7, 2, 13, 2, 5, 3, 2, 11, 2, 64, 2, 9)):
    """Portions of changing size, down to two tokens."""
    steps, s = [], 0
    for rid, toks in reqs.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}],
                          "end": [rid] if i + n == len(toks) else []})
            i += n
            s += 1
    return steps


def mixed(reqs, prompt_lens, max_live=4, chunk=(5, 9, 2, 16, 3), seed=0):
    """Up to ``max_live`` live requests: portions of some prompts beside single decoded
    tokens of others; a request starts when another has ended, so freed pages are used again.
    ``prompt_lens[rid]``: how much of the request counts as its prompt (run in portions);
    the rest runs one token per step."""
    rng = np.random.default_rng(seed)
    pending = list(reqs.items())
    live, done_at = {}, {}
    steps, s, k = [], 0, 0
    while pending or live:
        while pending and len(live) < max_live:
            rid, toks = pending.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            toks, i = reqs[rid], live[rid]
            if i < prompt_lens[rid]:
                if rng.random() < 0.25 and len(live) > 1:
                    continue                      # left out of this step, goes on later
                n = min(chunk[k % len(chunk)], prompt_lens[rid] - i)
                k += 1
            else:
                n = 1
            entries.append({"id": rid, "tokens": toks[i:i + n], "want": list(range(n))})
            live[rid] = i + n
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        steps.append({"step": s, "entries": entries, "end": end})
        s += 1
    return steps


def max_live_tokens(steps, round_to=64):
    """The most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held, best = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        best = max(best, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return best


def to_lines(steps):
    return io.StringIO("".join(json.dumps(st) + "\n" for st in steps))


def collect(steps, out_dir, vocab):
    """{request: [len, vocab] logits} from the files a replay wrote."""
    rows = {}
    for st in steps:
        n_want = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, f"{st['step']}.f32")
        if n_want == 0:
            assert not os.path.exists(path)
            continue
        data = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        r = 0
        for e in st["entries"]:
            for _ in e["want"]:
                rows.setdefault(e["id"], []).append(data[r])
                r += 1
    return {rid: np.stack(v) for rid, v in rows.items()}
