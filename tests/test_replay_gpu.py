"""Trace replay on the GPU against the plain implementation, in 32-bit and in bfloat16:
the same requests whole, with the last 32 tokens one by one, in portions of changing
size, and mixed with other requests in a pool so small that pages are used again."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_llama as P
import traces
from tiny import MAKE, logit_error, make_model, prompt_ids

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# fraction of the mean logit range: (max, mean)
TOL = {"float32": (1e-5, 1e-6), "bfloat16": (1e-2, 1e-3)}
WORKLOAD = {
    # prompt lengths and given decoded tokens (the two tiny workloads, plus lengths that
    # end exactly on a page and a long request)
    "A": ([5, 17, 33, 64, 150], 16),
    "B": ([1, 9, 40, 64, 100], 24),
    "C": ([3, 31, 70], 40),
    "D": ([200, 70, 640], 34),       # (from 512 rows the q/k/v product rotates and caches its own result)
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for which in WORKLOAD:
        d = make_model(which, str(tmp_path_factory.mktemp("model" + which)))
        cfg, w = P.load_folder(d)
        lens, extra = WORKLOAD[which]
        reqs = {f"r{i}": prompt_ids(n + extra, cfg["vocab_size"], 100 + i) for i, n in enumerate(lens)}
        plens = {f"r{i}": n for i, n in enumerate(lens)}
        want = {rid: P.forward(cfg, w, toks) for rid, toks in reqs.items()}
        out[which] = (d, cfg, reqs, plens, want)
    return out


def run_replay(model_dir, dtype, steps, tmp_path, page_size, max_tokens=None):
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    mt = max_tokens or traces.max_live_tokens(steps, max(64, page_size))
    runner = ModelRunner.from_folder(model_dir, dtype=dtype, max_tokens=mt, page_size=page_size, max_requests=4)
    out = str(tmp_path / "out")
    import io
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    runner.manager.check()
    assert not runner.manager.requests and runner.manager.free_pages() == runner.manager.pages_per_group
    return out, runner


def check(got, want, dtype, what):
    assert set(got) == set(want)
    for rid in want:
        assert got[rid].shape == want[rid].shape, (what, rid)
        assert np.abs(got[rid]).max() > 0, "all-zero logits"
        mx, mean = logit_error(got[rid], want[rid])
        tmax, tmean = TOL[dtype]
        if not (mx <= tmax and mean <= tmean):
            d = np.abs(got[rid] - want[rid]).max(axis=1)
            first = int(np.argmax(d > tmax * float(np.mean(want[rid].max(-1) - want[rid].min(-1)))))
            raise AssertionError(f"{what} {dtype} request {rid}: max {mx:.3e} mean {mean:.3e} of the logit range "
                                 f"(allowed {tmax:.0e} / {tmean:.0e}); first wrong position {first}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_schedules_match_plain(models, tmp_path, which, dtype, schedule):
    d, cfg, reqs, plens, want = models[which]
    page_size = {"A": 16, "B": 64, "C": 4, "D": 64}[which]
    if schedule == "whole":
        steps = traces.whole(reqs)
    elif schedule == "tail":
        steps = traces.tail_one_by_one(reqs, 32)
    elif schedule == "portions":
        steps = traces.portions(reqs)
    else:
        steps = traces.mixed(reqs, plens, max_live=4 if which != "A" else 3, seed=len(which))
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size)
    got = traces.collect(steps, out, cfg["vocab_size"])
    check(got, want, dtype, f"{which}/{schedule}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_of_several_requests_in_one_step(models, tmp_path, dtype):
    """A step of more than 512 rows made of three requests: one that goes on at a position that
    is no multiple of 8, one whole prompt, one decoded token between them.  The kernels that take
    many rows at once (tile products, the product that rotates and caches its own result, 128-row
    attention blocks) see request edges and groups of 8 positions that are not whole."""
    d, cfg, reqs, plens, want = models["D"]
    a, b, c = reqs["r2"], reqs["r0"], reqs["r1"]
    steps = [
        {"step": 0, "entries": [{"id": "r2", "tokens": a[:3], "want": [0, 1, 2]},
                                {"id": "r1", "tokens": c[:50], "want": list(range(50))}], "end": []},
        {"step": 1, "entries": [{"id": "r2", "tokens": a[3:333], "want": list(range(330))},
                                {"id": "r1", "tokens": c[50:51], "want": [0]},
                                {"id": "r0", "tokens": b, "want": list(range(len(b)))}], "end": ["r0"]},
        {"step": 2, "entries": [{"id": "r1", "tokens": c[51:], "want": list(range(len(c) - 51))},
                                {"id": "r2", "tokens": a[333:], "want": list(range(len(a) - 333))}], "end": ["r1", "r2"]},
    ]
    assert sum(len(e["tokens"]) for e in steps[1]["entries"]) >= 512
    out, runner = run_replay(d, dtype, steps, tmp_path, 64)
    check(traces.collect(steps, out, cfg["vocab_size"]), want, dtype, "D/long portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_are_used_again_and_old_contents_never_show(models, tmp_path, dtype):
    """The pool holds barely more than the live requests; every page is poisoned with NaN before
    the replay, so a read beyond a request's length, or of a page it does not own, shows."""
    import torch
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    import io
    d, cfg, reqs, plens, want = models["B"]
    steps = traces.mixed(reqs, plens, max_live=2, seed=5)
    mt = traces.max_live_tokens(steps, 64)
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=mt, page_size=8, max_requests=2)
    for lc in runner.storage.layers:
        lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    seen = set()
    orig_step = runner.step

    def spying_step(entries):
        r = orig_step(entries)
        for rc in runner.manager.requests.values():
            seen.update((id(rc), p) for p in rc.tables[0])
        return r
    runner.step = spying_step
    out = str(tmp_path / "o")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    pages_by_req = {}
    for rid, p in seen:
        pages_by_req.setdefault(p, set()).add(rid)
    assert any(len(v) > 1 for v in pages_by_req.values()), "no page was used by two requests"
    check(traces.collect(steps, out, cfg["vocab_size"]), want, dtype, "B/reuse")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user runs it: a child process, steps on stdin, 'done <step>' lines back."""
    d, cfg, reqs, plens, want = models["A"]
    steps = traces.mixed(reqs, plens, max_live=4, seed=9)
    # a step in which nothing is wanted writes no file
    steps[0]["entries"][0]["want"] = []
    mt = traces.max_live_tokens(steps, 64)
    out = str(tmp_path / "out")
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                          "--out", out, "--max-tokens", str(mt)], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                         text=True)
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {st['step']}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    got = traces.collect(steps, out, cfg["vocab_size"])
    first = steps[0]["entries"][0]
    n0 = len(first["tokens"])
    w = dict(want)
    w[first["id"]] = want[first["id"]][n0:]
    check(got, w, dtype, "trace_run")


def test_out_of_pages_is_an_error_that_changes_nothing(models):
    from xyntetik_runner_amd.cache import OutOfPages
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, reqs, plens, want = models["A"]
    runner = ModelRunner.from_folder(d, dtype="float32", max_tokens=64, page_size=16, max_requests=2)
    toks = reqs["r3"]
    runner.step([StepEntry("a", toks[:40], [])])
    free = runner.manager.free_pages()
    slots = runner.manager.slots.n_free
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", toks[40:60], []), StepEntry("b", toks[:30], [])])
    assert runner.manager.free_pages() == free and runner.length("a") == 40
    # the request the failed step would have started is not live and holds no state slot
    assert not runner.has("b") and runner.manager.slots.n_free == slots
    # nor does a step leave anything behind that asks for more state slots than there are
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("c", toks[:2], []), StepEntry("d", toks[:2], [])])
    assert not runner.has("c") and not runner.has("d") and runner.manager.slots.n_free == slots
    # or whose wanted places lie outside its tokens
    with pytest.raises(ValueError):
        runner.step([StepEntry("c", toks[:2], [2])])
    assert not runner.has("c") and runner.manager.free_pages() == free
    runner.manager.check()
    got = runner.step([StepEntry("a", toks[40:64], list(range(24)))]).cpu().numpy()
    mx, mean = logit_error(got, want["r3"][40:64])
    assert mx <= TOL["float32"][0]
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(models, tmp_path, dtype):
    """A short prompt and 250 tokens decoded one by one through the captured decode step:
    pages fill and new ones are taken, the attention's key ranges change, and every
    position still matches the plain implementation."""
    d, cfg, reqs, plens, want = models["A"]
    toks = prompt_ids(258, cfg["vocab_size"], 77)
    full = P.forward(cfg, *[P.load_folder(d)[1]], toks)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:8], "want": list(range(8))}], "end": []}]
    for i in range(8, len(toks)):
        steps.append({"step": i - 7, "entries": [{"id": "x", "tokens": [toks[i]], "want": [0]}],
                      "end": ["x"] if i == len(toks) - 1 else []})
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size=16)
    assert runner.graphs.replays >= 200 and runner.graphs.captures >= 2
    check(traces.collect(steps, out, cfg["vocab_size"]), {"x": full}, dtype, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(models, tmp_path, dtype):
    """Positions 0, 1, 2, ... of fresh requests: one token at a time, and two requests side by side."""
    d, cfg, reqs, plens, want = models["B"]
    w = P.load_folder(d)[1]
    a, b = prompt_ids(5, cfg["vocab_size"], 1), prompt_ids(5, cfg["vocab_size"], 2)
    steps = [{"step": i, "entries": [{"id": "a", "tokens": [a[i]], "want": [0]}, {"id": "b", "tokens": [b[i]], "want": [0]}],
              "end": ["a", "b"] if i == 4 else []} for i in range(5)]
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size=64)
    check(traces.collect(steps, out, cfg["vocab_size"]), {"a": P.forward(cfg, w, a), "b": P.forward(cfg, w, b)}, dtype, "first tokens")


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-6), ("bfloat16", 3e-3)])
def test_graph_and_eager_decode_agree(models, dtype, tol):
    """The captured decode step against the same step run kernel by kernel, replayed several
    times with other work between the replays.  The two split the keys of a request into
    ranges differently, so they agree to rounding, not bit for bit."""
    import torch
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, reqs, plens, want = models["A"]
    toks = reqs["r4"]
    outs = {}
    for use in (True, False):
        r = ModelRunner.from_folder(d, dtype=dtype, max_tokens=512, page_size=16, max_requests=4, use_graphs=use)
        r.step([StepEntry("p", toks[:40], []), StepEntry("q", toks[:17], [])])
        rows = []
        for i in range(40, 70):
            o = r.step([StepEntry("p", [toks[i]], [0]), StepEntry("q", [toks[i - 23]], [0])])
            rows.append(o.cpu().numpy())
            if i % 7 == 0:          # eager work between replays: a prompt portion of a third request
                r.step([StepEntry("z", toks[:9], [8])])
                r.finish("z")
        outs[use] = np.concatenate(rows)
        if use:
            assert r.graphs.replays >= 25
    mx, mean = logit_error(outs[True], outs[False])
    assert mx <= tol and np.abs(outs[True]).max() > 0, (mx, mean)


@pytest.mark.parametrize("which", ["A", "B"])
def test_decoding_with_norms_folded_into_the_products(models, which):
    """When few tokens are decoded in bfloat16, the norms between the products run inside the
    products' kernels.  The norm's own kernel is then launched twice a step (the first layer's
    first norm and the final norm) instead of 2 x layers + 1 times, and the logits agree with
    the separate kernels' to bfloat16 rounding and with the plain implementation as before."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, reqs, plens, want = models[which]
    toks = reqs["r3"]
    n0 = len(toks) - 12
    outs, launches = {}, {}
    for fold in (True, False):
        r = ModelRunner.from_folder(d, dtype="bfloat16", max_tokens=512, page_size=16, max_requests=4, use_graphs=False)
        count = [0]
        plain_norm = r.ops.rmsnorm
        def counting(*a, _f=plain_norm, _c=count, **k):
            _c[0] += 1
            return _f(*a, **k)
        try:                        # (the kernels' object is shared by every runner of the process)
            r.ops.fold_norms, r.ops.rmsnorm = fold, counting
            r.step([StepEntry("p", toks[:n0], []), StepEntry("q", toks[:7], [])])
            count[0] = 0
            rows = [r.step([StepEntry("p", [toks[i]], [0]), StepEntry("q", [toks[i - n0 + 7]], [])]).cpu().numpy()
                    for i in range(n0, len(toks))]
        finally:
            r.ops.fold_norms = True
            del r.ops.rmsnorm       # the instance attribute that hid the method
        outs[fold], launches[fold] = np.concatenate(rows), count[0] // 12
    L = cfg["num_hidden_layers"]
    assert launches == {True: 2, False: 2 * L + 1}
    for fold in (True, False):
        mx, mean = logit_error(outs[fold], want["r3"][n0:])
        assert mx <= TOL["bfloat16"][0] and mean <= TOL["bfloat16"][1], (fold, mx, mean)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_references_batch_workload(models, dtype):
    """The workload of the reference's own batching test (/root/reference/tests/test_batch.c:49-60,
    :203-215): 8 sequences with prompts of 5, 11, 8, 17, 6, 14, 9 and 20 tokens, ids
    ((seq+1)*7919 + i*104729) mod V, 24 greedy steps, decoded 1, 2, 4 and 8 at a time, so that
    every sequence of a batch sits at another position in every step.  Whole logits rows are
    compared, not only tokens, and they must not be all zero (its anti-vacuity rule)."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, _, _, _ = models["A"]
    _, w = P.load_folder(d)
    V, steps = cfg["vocab_size"], 24
    plen = [5, 11, 8, 17, 6, 14, 9, 20]
    prompts = [[((s + 1) * 7919 + i * 104729) % V for i in range(n)] for s, n in enumerate(plen)]
    full = [p + P.greedy(cfg, w, p, steps) for p in prompts]
    want = [P.forward(cfg, w, toks[:-1]) for toks in full]                  # row t: logits after token t
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=8 * 64, page_size=16, max_requests=8)
    for width in (1, 2, 4, 8):
        for g0 in range(0, 8, width):
            group = list(range(g0, g0 + width))
            got = {s: [] for s in group}
            out = runner.step([StepEntry(s, prompts[s], [plen[s] - 1]) for s in group])
            for r, s in enumerate(group):
                got[s].append(out[r].cpu().numpy())
            for k in range(steps - 1):
                out = runner.step([StepEntry(s, [full[s][plen[s] + k]], [0]) for s in group])
                for r, s in enumerate(group):
                    got[s].append(out[r].cpu().numpy())
            for s in group:
                rows = np.stack(got[s])
                assert np.abs(rows).max() > 0
                mx, mean = logit_error(rows, want[s][plen[s] - 1:])
                assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (width, s, mx, mean)
                if dtype == "float32":                                      # and the greedy tokens are the same
                    assert [int(np.argmax(r)) for r in rows] == full[s][plen[s]:]
                runner.finish(s)
        runner.manager.check()
        assert runner.manager.free_pages() == runner.manager.pages_per_group


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [1, 2])
def test_the_smallest_pages(models, tmp_path, dtype, page_size):
    """Pages of one and of two positions: every key has its own entry in the block table."""
    d, cfg, reqs, plens, want = models["A"]
    few = {rid: reqs[rid] for rid in ("r0", "r1", "r2")}
    steps = traces.mixed(few, plens, max_live=3, seed=page_size)
    out, runner = run_replay(d, dtype, steps, tmp_path, page_size)
    check(traces.collect(steps, out, cfg["vocab_size"]), {rid: want[rid] for rid in few}, dtype, f"pages of {page_size}")
