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


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_schedules_in_32_bit(models, tmp_path, seed):
    """Mixed schedules drawn at random (portion sizes, how many requests are live, which are left out of
    a step, the page size), in 32-bit where any fault of the cache or the batch shows above rounding."""
    rng = np.random.default_rng(seed)
    which = ["A", "B", "C"][seed % 3]
    d, cfg, reqs, plens, want = models[which]
    chunk = tuple(int(n) for n in rng.integers(2, 40, size=5))
    page_size = int(rng.choice([2, 4, 8, 16, 32, 64]))
    steps = traces.mixed(reqs, plens, max_live=int(rng.integers(2, 5)), chunk=chunk, seed=seed)
    out, runner = run_replay(d, "float32", steps, tmp_path, page_size)
    check(traces.collect(steps, out, cfg["vocab_size"]), want, "float32", f"{which}/random {seed}, pages of {page_size}, portions {chunk}")


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


def poison(runner):
    """Every page of every layer holds NaN: a read beyond a request's length, or of a page it does
    not own, shows in the logits."""
    for lc in runner.storage.layers:
        if lc.owns and lc.k is not None:
            lc.k.fill_(float("nan"))
            lc.v.fill_(float("nan"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,page_size", [("B", 8), ("B", 16), ("B", 64), ("D", 16), ("D", 64)])
def test_pages_are_used_again_and_old_contents_never_show(models, tmp_path, dtype, which, page_size):
    """The pool holds barely more than the live requests and every page is poisoned with NaN before
    the replay.  With pages of 8 positions bfloat16 attention is the 32-bit-arithmetic kernel; with 16
    and 64 it is the matrix-core kernels (decoded tokens and short portions, and for the longer
    requests of model D the 128-row blocks) and the products that rotate and cache their own result
    (src/engine.c:218-221: a cached row is a function of its request's own tokens only)."""
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    import io
    d, cfg, reqs, plens, want = models[which]
    steps = traces.mixed(reqs, plens, max_live=2, seed=5)
    mt = traces.max_live_tokens(steps, max(64, page_size))
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=mt, page_size=page_size, max_requests=2)
    poison(runner)
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
    check(traces.collect(steps, out, cfg["vocab_size"]), want, dtype, f"{which}/reuse, pages of {page_size}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which,page_size", [("A", 16), ("B", 64), ("D", 64)])
def test_which_pages_a_request_gets_does_not_matter(models, tmp_path, dtype, which, page_size):
    """The same mixed trace twice, in a pool three times the size it needs: once with the free list
    as it is made (lowest page first), once shuffled, so that every request's pages lie scattered
    and in another order.  A page number is an address and nothing else (tests/test_prefix.c:17-20:
    rows land where the table says and read back the same), so the logits are the same to the bit."""
    import random
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    import io
    d, cfg, reqs, plens, want = models[which]
    steps = traces.mixed(reqs, plens, max_live=3, seed=11)
    mt = 3 * traces.max_live_tokens(steps, max(64, page_size))
    got, tables = {}, {}
    for shuffled in (False, True):
        runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=mt, page_size=page_size, max_requests=3)
        poison(runner)
        if shuffled:
            for g in runner.manager.groups:
                random.Random(17).shuffle(g.pool._free)
        used = []
        orig_step = runner.step

        def spying_step(entries, _orig=orig_step, _runner=runner, _used=used):
            r = _orig(entries)
            _used.append(sorted((str(rc.req_id), tuple(rc.tables[0])) for rc in _runner.manager.requests.values()))
            return r
        runner.step = spying_step
        out = str(tmp_path / f"o{int(shuffled)}")
        replay(runner, traces.to_lines(steps), out, report=io.StringIO())
        runner.manager.check()
        got[shuffled], tables[shuffled] = traces.collect(steps, out, cfg["vocab_size"]), used
    assert tables[True] != tables[False], "the shuffled free list gave the same pages"
    check(got[False], want, dtype, f"{which}/pages in order")
    for rid in want:
        assert np.array_equal(got[True][rid], got[False][rid]), f"request {rid}: logits depend on the page numbers"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_that_fails_leaves_the_recorded_steps_tables_right(models, dtype):
    """Two requests decode through a recorded step and both take a new page in the same step; that
    step fails after its block tables have gone to the device.  The pages it reserved go back, and the
    next step hands them out the other way round (the page given back last is taken first): the
    recorded step's copy of the tables must follow, or each request reads the other's page."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, reqs, plens, want = models["A"]
    a, b = reqs["r3"], reqs["r4"]                     # 80 and 166 tokens
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=512, page_size=16, max_requests=2)
    runner.step([StepEntry("a", a[:14], []), StepEntry("b", b[:30], [])])
    got = {"a": [], "b": []}

    def decode(i):
        out = runner.step([StepEntry("a", [a[14 + i]], [0]), StepEntry("b", [b[30 + i]], [0])]).cpu().numpy()
        got["a"].append(out[0]); got["b"].append(out[1])
    decode(0); decode(1)                              # lengths 16 and 32: the next token of each opens a page
    assert runner.graphs.captures >= 1
    before = {r: list(runner.manager.get(r).tables[0]) for r in "ab"}
    run = runner.graphs.run

    def fails_after_the_tables_are_copied(*args, **kw):
        run(*args, **kw)
        raise RuntimeError("injected")
    runner.graphs.run = fails_after_the_tables_are_copied
    with pytest.raises(RuntimeError, match="injected"):
        decode(2)
    runner.graphs.run = run
    assert {r: list(runner.manager.get(r).tables[0]) for r in "ab"} == before and runner.length("a") == 16
    runner.manager.check()
    for i in range(2, 20):
        decode(i)
    runner.manager.check()
    for rid, toks, n0 in (("a", a, 14), ("b", b, 30)):
        mx, mean = logit_error(np.stack(got[rid]), want["r3" if rid == "a" else "r4"][n0:n0 + 20])
        assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (rid, mx, mean)


WIDE = {"A": 16, "B": 64, "D": 64}       # page sizes


@pytest.fixture(scope="module")
def wide(models):
    """64 requests for each of three models: prompts of 1 to 150 tokens and 8 to 32 given decoded
    tokens, with the plain logits of every place."""
    out = {}
    for which in WIDE:
        d, cfg, _, _, _ = models[which]
        _, w = P.load_folder(d)
        rng = np.random.default_rng(40 + len(out))
        plen = [int(n) for n in rng.integers(1, 151, size=64)]
        plen[0], plen[1], plen[2] = 1, 150, 64
        ndec = [8 + int(n) for n in rng.integers(0, 25, size=64)]
        ndec[0], ndec[5] = 32, 8
        toks = [prompt_ids(plen[i] + ndec[i], cfg["vocab_size"], 900 + i) for i in range(64)]
        want = [P.forward(cfg, w, t, all_at_once=True) for t in toks]
        out[which] = (d, cfg, plen, ndec, toks, want)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "D"])
def test_three_hundred_requests_decode_in_the_largest_recorded_step(models, which, dtype):
    """300 requests with prompts of 1 to 6 tokens decode 5 tokens each side by side: the recorded step
    for 512 rows (212 pad it), in which the q/k/v product is a tile product that rotates and caches its
    own result from one table of the step's cosines and sines that all layers share inside the recording."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, _, _, _ = models[which]
    _, w = P.load_folder(d)
    n, n_dec = 300, 5
    rng = np.random.default_rng(8)
    plen = [int(x) for x in rng.integers(1, 7, size=n)]
    toks = [prompt_ids(plen[i] + n_dec, cfg["vocab_size"], 3000 + i) for i in range(n)]
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=n * 64, page_size=16, max_requests=n)
    poison(runner)
    for g0 in range(0, n, 50):
        runner.step([StepEntry(i, toks[i][:plen[i]], []) for i in range(g0, g0 + 50)])
    got = {i: [] for i in range(n)}
    for k in range(n_dec):
        out = runner.step([StepEntry(i, [toks[i][plen[i] + k]], [0]) for i in range(n)]).cpu().numpy()
        for i in range(n):
            got[i].append(out[i])
    assert runner.graphs.captures == 1 and runner.graphs.replays == n_dec - 1
    for i in range(n):
        rows = np.stack(got[i])
        want = P.forward(cfg, w, toks[i], all_at_once=True)[plen[i]:]
        assert np.isfinite(rows).all() and np.abs(rows).max() > 0
        mx, mean = logit_error(rows, want)
        assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (which, dtype, i, plen[i], mx, mean)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_live", [20, 40, 64])
@pytest.mark.parametrize("which", list(WIDE))
def test_many_requests_decode_through_recorded_steps(wide, which, n_live, dtype):
    """20, 40 and 64 requests decode side by side (tests/test_batch.c:49-60, :203-215, past its 8):
    the recorded steps for 32 and 64 rows, whose products take the kernels for 17 to 64 rows, with
    rows that pad the batch (12 and 24 from the first step on, more as requests end at different
    times), requests of 1 to 150 prompt tokens at different positions in every step, and every row
    of every step against the plain implementation."""
    from xyntetik_runner_amd.engine.batch import StepEntry
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, plen, ndec, toks, want = wide[which]
    ps = WIDE[which]
    ids = list(range(n_live))
    mt = sum(-(-(plen[i] + ndec[i]) // max(64, ps)) * max(64, ps) for i in ids)
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=mt, page_size=ps, max_requests=n_live)
    poison(runner)
    got = {i: [] for i in ids}
    for g0 in range(0, n_live, 7):                    # the prompts, 7 requests a step
        group = ids[g0:g0 + 7]
        out = runner.step([StepEntry(i, toks[i][:plen[i]], list(range(plen[i]))) for i in group]).cpu().numpy()
        r = 0
        for i in group:
            got[i].append(out[r:r + plen[i]])
            r += plen[i]
    assert runner.graphs.replays == 0 and runner.graphs.captures == 0
    n_steps, widths = 0, set()
    for k in range(max(ndec[i] for i in ids)):
        live = [i for i in ids if k < ndec[i]]
        out = runner.step([StepEntry(i, [toks[i][plen[i] + k]], [0]) for i in live]).cpu().numpy()
        widths.add(len(live))
        n_steps += 1
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
            if k == ndec[i] - 1:
                runner.finish(i)
    assert n_steps >= 24 and len(widths) > 3, "the batch never shrank"
    # every decode step went through a recorded step (its first run records it)
    assert runner.graphs.replays + runner.graphs.captures == n_steps and runner.graphs.replays > n_steps // 2
    runner.manager.check()
    assert runner.manager.all_free()
    for i in ids:
        rows = np.concatenate(got[i])
        assert rows.shape == want[i].shape and np.isfinite(rows).all() and np.abs(rows).max() > 0
        mx, mean = logit_error(rows, want[i])
        if not (mx <= TOL[dtype][0] and mean <= TOL[dtype][1]):
            dd = np.abs(rows - want[i]).max(axis=1)
            raise AssertionError(f"{which} {dtype} {n_live} live, request {i} (prompt {plen[i]}): max {mx:.3e} mean "
                                 f"{mean:.3e}; worst place {int(dd.argmax())}")


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
    """The workload of the reference's own batching test (tests/test_batch.c:49-60,
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
