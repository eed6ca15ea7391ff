"""Generation on the GPU: greedy and sampled decoding through the entry points, the
sampling kernel against the plain sampler, preemption, and the command line."""
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_llama as P
from tiny import make_model, prompt_ids

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {w: make_model(w, str(tmp_path_factory.mktemp("gen" + w))) for w in ("A", "B")}


def near_argmax(cfg, w, prompt, out, frac):
    """Every generated token is the plain model's argmax for its prefix, or within ``frac`` of the range of it."""
    toks = list(prompt)
    for t in out:
        lg = P.forward(cfg, w, toks)[-1]
        assert lg.max() - lg[t] <= frac * (lg.max() - lg.min()), (len(toks), t, int(lg.argmax()))
        toks.append(t)


@pytest.mark.parametrize("which,lens,n_new", [("A", [5, 17, 33], 16), ("B", [1, 9, 40, 64, 100], 24)])
def test_greedy_through_the_entry_point(folders, which, lens, n_new):
    from xyntetik_runner_amd import LLM, SamplingParams
    cfg, w = P.load_folder(folders[which])
    prompts = [prompt_ids(n, cfg["vocab_size"], 50 + i) for i, n in enumerate(lens)]
    llm = LLM(folders[which], dtype="float32", max_tokens=1024, page_size=16, max_batched_tokens=48)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=n_new))
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        assert o == P.greedy(cfg, w, p, n_new)
    llm.runner.manager.check()
    del llm
    llm = LLM(folders[which], dtype="bfloat16", max_tokens=1024, page_size=64, max_batched_tokens=64)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=n_new))
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        near_argmax(cfg, w, p, o, 0.02)


def test_the_cache_is_sized_from_the_card_by_default(folders, tmp_path):
    """A model whose config names a context of 131,072 (as the real Llama-3.1 files do) loads through
    the entry point with nothing said about the cache: the pool takes what 64 requests of that length
    need or what 90% of the card leaves, whichever is less, one request of the whole context fits, and
    generation works.  With almost no memory allowed the error says what is missing
    (src/model.h:516-592: the reference caps the context it allocates)."""
    import json
    import shutil
    import torch
    from xyntetik_runner_amd import LLM, SamplingParams
    from xyntetik_runner_amd.cache import CacheTooSmall
    d = str(tmp_path / "long_context")
    shutil.copytree(folders["A"], d)
    with open(os.path.join(d, "config.json")) as f:
        cfg = json.load(f)
    cfg["max_position_embeddings"] = 131072
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    llm = LLM(d, dtype="bfloat16")
    m = llm.runner.manager
    free, total = torch.cuda.mem_get_info()
    assert 131072 <= m.capacity_tokens() <= 64 * 131072
    assert llm.runner.storage.bytes_per_token() * m.capacity_tokens() <= 0.9 * total
    _, w = P.load_folder(folders["A"])
    prompt = prompt_ids(19, 256, 4)
    out = llm.generate([prompt], SamplingParams(max_new_tokens=6))[0]
    near_argmax(cfg, w, prompt, out, 0.02)
    del llm
    with pytest.raises(CacheTooSmall, match="does not hold one request of 131072 tokens"):
        LLM(d, dtype="bfloat16", gpu_memory_fraction=1e-6)
    # an explicit number of tokens is taken as it is
    llm = LLM(d, dtype="bfloat16", max_tokens=512)
    assert llm.runner.manager.capacity_tokens() == 512


def test_sampled_tokens_depend_on_the_request_alone(folders):
    from xyntetik_runner_amd import LLM, SamplingParams
    cfg, w = P.load_folder(folders["B"])
    prompts = [prompt_ids(n, 384, 70 + i) for i, n in enumerate([1, 9, 40, 64, 100])]
    sp = [SamplingParams(temperature=0.8, seed=1000 + i, max_new_tokens=24) for i in range(5)]
    llm = LLM(folders["B"], dtype="float32", max_tokens=2048, page_size=16, max_batched_tokens=32)
    together = llm.generate(prompts, sp)
    again = llm.generate(prompts, sp)
    assert together == again
    alone = [llm.generate([p], s)[0] for p, s in zip(prompts, sp)]
    assert alone == together
    other_seed = llm.generate(prompts[2:3], SamplingParams(temperature=0.8, seed=5, max_new_tokens=24))[0]
    assert other_seed != together[2]
    # each token is what the plain sampler picks from the plain logits with the same draw
    for p, s, out in zip(prompts, sp, together):
        state, toks = s.seed, list(p)
        for t in out:
            state, r = P.rng_f32(state)
            assert P.sample_pick(P.forward(cfg, w, toks)[-1], 0.8, r) == t
            toks.append(t)


def test_sampling_kernel_matches_plain_sampler():
    import torch
    from xyntetik_runner_amd.csrc.ops import load_ops
    ops = load_ops()
    rng = np.random.default_rng(0)
    cases = []
    for V in (8, 333, 5000):
        for _ in range(6):
            lg = (rng.normal(size=V) * rng.choice([0.5, 3.0])).astype(np.float32)
            if rng.random() < 0.5:
                lg[rng.integers(0, V, size=V // 3)] = lg[0]             # exact ties
            kw = dict(temp=float(rng.choice([0.0, 0.3, 0.8, 1.5])), draw=float(np.float32(rng.random())),
                      top_k=int(rng.choice([0, 1, 5, 40])), top_p=float(rng.choice([1.0, 0.9, 0.5])),
                      min_p=float(rng.choice([0.0, 0.05, 0.3])), repeat_penalty=float(rng.choice([1.0, 1.3])),
                      recent=[int(t) for t in rng.integers(-2, V + 2, size=rng.integers(0, 20))])
            cases.append((V, lg, kw))
    all_equal = np.full(64, 1.25, dtype=np.float32)
    cases.append((64, all_equal, dict(temp=1.0, draw=0.5, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, recent=[])))
    cases.append((64, all_equal, dict(temp=1.0, draw=0.99, top_k=10, top_p=1.0, min_p=0.0, repeat_penalty=1.0, recent=[])))
    cases.append((64, all_equal, dict(temp=0.0, draw=0.99, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, recent=[])))
    # the reference's own penalty vector (tests/test_sampler.c:200-206): token 1
    cases.append((4, np.array([10.0, 9.0, 1.0, 0.5], dtype=np.float32),
                  dict(temp=0.01, draw=0.7, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=2.0, recent=[0])))
    exempt = [3]
    for V, lg, kw in cases:
        want = P.sample_pick(lg, kw["temp"], kw["draw"], kw["top_k"], kw["top_p"], kw["min_p"],
                             kw["repeat_penalty"], kw["recent"], exempt)
        dev = torch.device("cuda:0")
        rec = torch.zeros((1, 256), dtype=torch.int32)
        rec[0, :len(kw["recent"])] = torch.tensor(kw["recent"], dtype=torch.int32)
        t = torch.tensor(lg, device=dev).unsqueeze(0).contiguous()
        before = t.clone()
        got = ops.sample(t, torch.tensor([kw["temp"]], device=dev), torch.tensor([kw["draw"]], device=dev),
                         top_k=torch.tensor([kw["top_k"]], dtype=torch.int32, device=dev),
                         top_p=torch.tensor([kw["top_p"]], device=dev), min_p=torch.tensor([kw["min_p"]], device=dev),
                         repeat_penalty=torch.tensor([kw["repeat_penalty"]], device=dev), recent=rec.to(dev),
                         n_recent=torch.tensor([len(kw["recent"])], dtype=torch.int32, device=dev),
                         exempt=torch.tensor(exempt, dtype=torch.int32, device=dev))
        assert int(got[0]) == want, (V, kw, int(got[0]), want)
        if kw["temp"] <= 0:
            assert torch.equal(t, before)                              # greedy leaves the logits untouched


def test_sampling_kernel_distribution_and_many_rows():
    import torch
    from xyntetik_runner_amd.csrc.ops import load_ops
    ops = load_ops()
    dev = torch.device("cuda:0")
    V, n = 8192, 4000
    lg = np.full(V, -20.0, dtype=np.float32)
    lg[[5, 100, 4000]] = [6.0, 5.4, 4.8]
    z = np.exp(lg.astype(np.float64)); z /= z.sum()
    s, draws = 42, []
    for _ in range(n):
        s, r = P.rng_f32(s)
        draws.append(r)
    rows = torch.tensor(lg, device=dev).repeat(n, 1).contiguous()
    got = ops.sample(rows, torch.ones(n, device=dev), torch.tensor(draws, dtype=torch.float32, device=dev)).cpu().numpy()
    for t in (5, 100, 4000):
        assert abs((got == t).mean() - z[t]) < 0.03
    mixed_t = torch.tensor([0.0, 1.0] * (n // 2), device=dev)
    got2 = ops.sample(rows, mixed_t, torch.tensor(draws, dtype=torch.float32, device=dev)).cpu().numpy()
    assert np.all(got2[0::2] == 5) and np.array_equal(got2[1::2], got[1::2])
    # a temperature near zero picks like greedy whatever is drawn (tests/test_sampler.c:200-206)
    cold = ops.sample(rows, torch.full((n,), 0.01, device=dev), torch.tensor(draws, dtype=torch.float32, device=dev))
    assert np.all(cold.cpu().numpy() == 5)


def test_greedy_pick_over_a_long_row_split_in_ranges():
    """Long rows are read by several workgroups: the first index of the maximum must still win,
    wherever the ties fall, and rows with temperature beside them are left to the sampler."""
    import torch
    from xyntetik_runner_amd.csrc.ops import load_ops
    ops = load_ops()
    dev = torch.device("cuda:0")
    V = 50001                                             # no multiple of the 32 ranges, nor of 4
    rng = np.random.default_rng(3)
    rows = rng.normal(size=(7, V)).astype(np.float32)
    chunk = ((V + 31) // 32 + 3) & ~3
    rows[0, [chunk - 1, chunk, 3 * chunk + 5, V - 1]] = 9.0   # ties on both sides of a range's edge and at the end
    rows[1, V - 1] = 9.0                                   # the last element alone
    rows[2, :] = -np.inf                                   # nothing is larger than anything: index 0
    rows[3, :] = np.nan
    rows[3, 40000] = -5.0                                  # the only number
    rows[4, 0] = 9.0
    rows[5, [17, 30000]] = [8.0, 9.0]
    t = torch.tensor(rows, device=dev)
    temp = torch.zeros(7, device=dev)
    temp[6] = 1.0
    rows[6, :] = -30.0
    rows[6, 123] = 30.0                                    # a sampled row with one token that has all the mass
    t[6] = torch.tensor(rows[6], device=dev)
    got = ops.sample(t, temp, torch.full((7,), 0.5, device=dev)).cpu().tolist()
    assert got == [chunk - 1, V - 1, 0, 40000, 0, 30000, 123]


def test_preemption_gives_the_same_tokens(folders):
    """A pool too small for all requests at once: some are preempted and recomputed, and
    every request still gets the tokens it gets when it has the cache to itself."""
    from xyntetik_runner_amd import LLM, SamplingParams
    cfg, w = P.load_folder(folders["A"])
    prompts = [prompt_ids(n, 256, 90 + i) for i, n in enumerate([30, 22, 41, 9])]
    sp = [SamplingParams(temperature=0.7 if i % 2 else 0.0, seed=77 + i, max_new_tokens=40) for i in range(4)]
    big = LLM(folders["A"], dtype="float32", max_tokens=1024, page_size=8, max_batched_tokens=24)
    want = big.generate(prompts, sp)
    assert big.engine.stats.preemptions == 0
    small = LLM(folders["A"], dtype="float32", max_tokens=160, page_size=8, max_batched_tokens=24)
    got = small.generate(prompts, sp)
    assert small.engine.stats.preemptions > 0
    assert got == want
    small.runner.manager.check()
    assert small.runner.manager.free_pages() == small.runner.manager.pages_per_group


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_queued_ahead_change_nothing(folders, dtype):
    """In steady decoding the engine queues the next step before it has read this step's tokens.
    Requests that end on a stop token (known one step late: that step's row is dropped), on
    their length, a request that joins meanwhile, sampled and greedy rows: every request gets
    the tokens it gets from an engine that never runs ahead, and every page comes back."""
    from xyntetik_runner_amd.engine import Engine, ModelRunner
    from xyntetik_runner_amd.sampling import SamplingParams
    cfg, w = P.load_folder(folders["A"])
    prompts = [prompt_ids(n, 256, 40 + i) for i, n in enumerate([9, 17, 30, 12, 21])]
    refs = [P.greedy(cfg, w, p, 14) for p in prompts[:2]]
    # a stop token that ends request 0 in the middle of its decoding (the others may hit it too:
    # whatever it does, both engines must agree)
    stop = next(t for k, t in enumerate(refs[0]) if k >= 4 and t not in refs[0][:k])
    params = [SamplingParams(max_new_tokens=30), SamplingParams(max_new_tokens=11),
              SamplingParams(temperature=0.8, seed=5, max_new_tokens=25),
              SamplingParams(temperature=0.6, top_k=20, seed=9, max_new_tokens=18),
              SamplingParams(max_new_tokens=16, ignore_eos=True)]
    results, ahead_steps = {}, {}
    for ahead in (False, True):
        runner = ModelRunner.from_folder(folders["A"], dtype=dtype, max_tokens=1024, page_size=16, max_requests=8)
        eng = Engine(runner, stop_ids=[stop], run_ahead=ahead)
        ids = [eng.add_request(p, sp) for p, sp in zip(prompts[:4], params[:4])]
        done, ended, steps = {}, {}, 0
        while eng.has_work():
            for o in eng.step():
                done.setdefault(o.req_id, []).append(o.token)
                if o.finished:
                    ended[o.req_id] = o.request
            steps += 1
            if steps == 6:                          # decoding is under way: a fifth request joins
                ids.append(eng.add_request(prompts[4], params[4]))
        assert not eng.requests                     # a request that has ended is the caller's, not the engine's
        results[ahead] = [list(ended[i].output) for i in ids]
        ahead_steps[ahead] = eng.stats.steps_ahead
        for i, rid in enumerate(ids):
            assert [t for t in done[rid] if t is not None] == results[ahead][i]
        runner.manager.check()
        assert not runner.manager.requests and runner.manager.free_pages() == runner.manager.pages_per_group
    assert ahead_steps[False] == 0 and ahead_steps[True] >= 10
    if dtype == "bfloat16":
        # A request that ended still has its row in the step queued ahead, so batches differ in size
        # between the two engines, and with them the order of some 32-bit sums: in bfloat16 a pick
        # near a boundary may then differ.  Until anything ended, the tokens are the same.
        assert [r[:5] for r in results[True]] == [r[:5] for r in results[False]]
        return
    assert results[True] == results[False]
    if dtype == "float32":
        first = refs[0].index(stop)
        assert results[True][0] == refs[0][:first]              # the stop token is not kept
        r1 = refs[1][:11]
        assert results[True][1] == (r1[:r1.index(stop)] if stop in r1 else r1)
    assert len(results[True][4]) == 16


def test_an_engine_is_used_again_and_a_request_is_aborted_while_a_step_is_queued_ahead(folders):
    """Generations one after the other on one engine (a step queued ahead for requests that have
    all ended is forgotten), and a request taken out between two steps while the next step,
    with its row in it, is already queued: the others go on as if it had never been there."""
    from xyntetik_runner_amd.engine import Engine, ModelRunner
    from xyntetik_runner_amd.sampling import SamplingParams
    cfg, w = P.load_folder(folders["A"])
    prompts = [prompt_ids(n, 256, 60 + i) for i, n in enumerate([11, 23, 8])]
    refs = [P.greedy(cfg, w, p, 12) for p in prompts]
    runner = ModelRunner.from_folder(folders["A"], dtype="float32", max_tokens=512, page_size=16, max_requests=4)
    eng = Engine(runner, stop_ids=[])
    sp = SamplingParams(max_new_tokens=12)
    assert eng.generate(prompts[:2], sp) == refs[:2]
    assert eng.generate(prompts[1:], sp) == refs[1:]                  # again, with what the first left behind
    assert eng.stats.steps_ahead > 0
    ids = [eng.add_request(p, sp) for p in prompts]
    for _ in range(5):
        eng.step()
    assert eng._ahead is not None                                     # a step with all three rows is on its way
    ended = {ids[1]: eng.abort(ids[1])}
    while eng.has_work():
        ended.update((o.req_id, o.request) for o in eng.step() if o.finished)
    assert [ended[i].output for i in (ids[0], ids[2])] == [refs[0], refs[2]]
    assert len(ended[ids[1]].output) < 12 and ended[ids[1]].finish_reason == "aborted" and not eng.requests
    runner.manager.check()
    assert not runner.manager.requests and runner.manager.free_pages() == runner.manager.pages_per_group


def test_stop_token_ends_a_request(folders):
    from xyntetik_runner_amd.engine import Engine, ModelRunner
    from xyntetik_runner_amd.sampling import SamplingParams
    cfg, w = P.load_folder(folders["A"])
    prompt = prompt_ids(12, 256, 3)
    ref = P.greedy(cfg, w, prompt, 10)
    runner = ModelRunner.from_folder(folders["A"], dtype="float32", max_tokens=256, page_size=16)
    eng = Engine(runner, stop_ids=[ref[4]])
    first = ref.index(ref[4])
    assert eng.generate([prompt], SamplingParams(max_new_tokens=10)) == [ref[:first]]    # the stop token is not kept
    eng = Engine(runner, stop_ids=[ref[4]])
    assert eng.generate([prompt], SamplingParams(max_new_tokens=10, ignore_eos=True)) == [ref]


def test_command_line(folders):
    cfg, w = P.load_folder(folders["A"])
    prompt = prompt_ids(7, 256, 11)
    want = P.greedy(cfg, w, prompt, 6)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "runner"), "-m", folders["A"], "--ids",
           ",".join(map(str, prompt)), "-n", "6", "--temp", "0", "--dtype", "float32"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    assert p.stdout.strip() == ",".join(map(str, prompt + want))
    assert "prompt: 7 tok" in p.stderr and "gen: 6 tok" in p.stderr
    # text prompt: bytes are ids; same seed gives the same text
    cmd = [sys.executable, os.path.join(ROOT, "bin", "runner"), "-m", folders["A"], "-p", "hi\\n", "-n", "5",
           "--temp", "0.9", "-s", "3", "--top-k", "50", "--dtype", "float32"]
    a = subprocess.run(cmd, capture_output=True, timeout=120)
    b = subprocess.run(cmd, capture_output=True, timeout=120)
    assert a.returncode == 0 and a.stdout == b.stdout and a.stdout.startswith(b"hi\n")
    bad = subprocess.run(cmd[:-2] + ["-s", "0"], capture_output=True, text=True, timeout=120)
    assert bad.returncode == 1 and "seed 0 cannot be used" in bad.stderr
    long = subprocess.run(cmd[:4] + ["--ids", ",".join(["1"] * 200), "-c", "100"], capture_output=True, text=True, timeout=120)
    assert long.returncode == 1 and "does not fit a context of 100" in long.stderr
