"""The serving benchmark: decode tokens a second for the Llama-3.1-8B shape with random
weights on one MI355X, plus the prefill rate at 2,048 tokens and the decode step's
fraction of the HBM roofline.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the engine (schedule, model step, sampling) for a batch of
8 requests, each with a 2,048-token prompt already in the cache.  One JSON line goes to
stdout.  The reference's own bench times a 512-token prompt and 128 greedy tokens of one
sequence and ignores end-of-text while it does (src/main.c:1435-1515).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LLAMA_3_1_8B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "intermediate_size": 14336, "vocab_size": 128256, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 8192, "hidden_act": "silu",
}
# other sizes of the same architecture (--shape); the default and the contract's line are the 8B shape
LLAMA_2_7B = dict(LLAMA_3_1_8B, num_key_value_heads=32, intermediate_size=11008, vocab_size=32000, rope_theta=10000.0,
                  rope_scaling=None, max_position_embeddings=4096)
LLAMA_3_1_70B = dict(LLAMA_3_1_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, intermediate_size=28672)
# a small shape of the same architecture with heads of 64 and tied embeddings (the sizes of a 1B-class Llama)
LLAMA_1B = dict(LLAMA_3_1_8B, num_hidden_layers=16, hidden_size=2048, head_dim=64, intermediate_size=8192,
                tie_word_embeddings=True, max_position_embeddings=131072,
                rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                              "original_max_position_embeddings": 8192})
SHAPES = {"llama-3.1-8b": ("Llama-3.1-8B shape", LLAMA_3_1_8B), "llama-2-7b": ("Llama-2-7B shape", LLAMA_2_7B),
          "llama-3.1-70b": ("Llama-3.1-70B shape", LLAMA_3_1_70B), "llama-1b-head64": ("Llama 1B-class shape, heads of 64", LLAMA_1B)}
PEAK = {"hbm_gbs": 8000.0, "bf16_flops": 2.5e15, "fp32_flops": 157.3e12}


def log(msg):
    sys.stderr.write(f"[bench] {msg}\n")
    sys.stderr.flush()


def build_runner(cfg, dtype, max_tokens, max_requests, seed=0):
    import torch
    from xyntetik_runner_amd.config import config_from_dict
    from xyntetik_runner_amd.engine import ModelRunner
    from xyntetik_runner_amd.engine.model import Model
    from xyntetik_runner_amd.weights import random_state
    arch, typed = config_from_dict(cfg)
    spec = arch.build_spec(typed)
    t0 = time.time()
    state = random_state(Model.expected_tensors(spec), seed, device=torch.device("cuda:0"))
    runner = ModelRunner(spec, state, dtype, max_tokens=max_tokens, page_size=64, max_requests=max_requests,
                         consume_state=True)      # the 70B shape is half the card: it must not stand there twice
    del state
    torch.cuda.synchronize()
    log(f"model with {len(spec.layers)} layers on the GPU in {time.time() - t0:.1f} s")
    return spec, runner


def matmul_params(cfg, layers):
    E, H, Hk, D, F, V = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                         cfg["intermediate_size"], cfg["vocab_size"])
    per_layer = E * (H * D + 2 * Hk * D) + H * D * E + 3 * E * F
    return per_layer * layers, V * E


def decode_bytes(cfg, layers, batch, ctx_tokens, elt=2):
    """Bytes one decode step has to read: every weight it uses once, and the cache of the live requests."""
    body, head = matmul_params(cfg, layers)
    norms = (2 * layers + 1) * cfg["hidden_size"]
    weights = (body + head + norms) * elt + batch * cfg["hidden_size"] * elt     # + one embedding row per request
    kv = ctx_tokens * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * layers * elt
    return weights + kv


def prefill_flops(cfg, layers, T):
    body, head = matmul_params(cfg, layers)
    attn = 4 * cfg["num_attention_heads"] * cfg["head_dim"] * layers * (T * (T + 1) // 2)
    return 2 * body * T + 2 * head * 1 + attn


def measure_achievable(runner):
    """What this GPU delivers to kernels with nothing else to do, as yardsticks beside the nominal
    peaks: bytes a second to a kernel that only reads (every workgroup a range of its own, 8 GB in
    all), and bfloat16 products a second of the matrix kernel on one large product of random data
    (8192 x 28672 x 4096).  The best of five each."""
    import torch
    ops = runner.ops
    dev = runner.device

    def best_ms(fn, reps=5):
        fn()
        best = None
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            b.synchronize()
            t = a.elapsed_time(b)
            best = t if best is None else min(best, t)
        return best
    n_bytes = 8 << 30
    buf = torch.empty((n_bytes,), dtype=torch.uint8, device=dev)
    buf.zero_()
    read_ms = best_ms(lambda: ops.stream_read(buf))
    del buf
    M, N, K = 8192, 28672, 4096
    a = (torch.randn((M, K), device=dev) * 0.5).bfloat16()
    w = ops.pack_weight((torch.randn((N, K), device=dev) * 0.02).bfloat16())
    out = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    mm_ms = best_ms(lambda: ops.linear(a, w, out=out))
    del a, w, out
    torch.cuda.empty_cache()
    return n_bytes / (read_ms * 1e-3) / 1e9, 2.0 * M * N * K / (mm_ms * 1e-3)


def measure_decode(runner, cfg, batch, prompt_len, steps, warmup, seed, alone=False):
    """tokens/s of `steps` decode steps with `batch` requests whose prompts are already cached;
    afterwards one more step's logits are checked (`check_decode_logits`)."""
    import numpy as np
    import torch
    from xyntetik_runner_amd.engine import Engine
    from xyntetik_runner_amd.sampling import SamplingParams
    # (prompts up to 8,192 tokens go in one step each, longer ones in portions of 2,048)
    budget = max(2048, prompt_len) if prompt_len <= 8192 else 2048
    eng = Engine(runner, max_batched_tokens=budget, max_running=batch,
                 max_model_len=cfg["max_position_embeddings"], stop_ids=[])
    rng = np.random.default_rng(seed)
    # a request admitted first decodes while the others' prompts are still computed (a step for
    # every portion of every prompt): nobody may finish before the last timed step
    sp = SamplingParams(temperature=0.0, max_new_tokens=batch * -(-prompt_len // budget) + warmup + steps + 8, ignore_eos=True)
    ids = [eng.add_request([int(t) for t in rng.integers(0, cfg["vocab_size"], size=prompt_len)], sp) for _ in range(batch)]
    def step():
        for o in eng.step():
            if o.finished:
                raise RuntimeError(f"decode batch {batch}: request {o.req_id!r} ended before the last timed step ({o.finish_reason})")
    while any(eng.requests[i].n_computed < prompt_len for i in ids):
        step()
    for _ in range(warmup):
        step()
    ctx0 = sum(eng.requests[i].n_tokens for i in ids)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    if len(eng.scheduler.running) != batch or any(i not in eng.requests for i in ids):
        raise RuntimeError(f"decode batch {batch}: a request ended or waited during the timed steps")
    ctx1 = sum(eng.requests[i].n_tokens for i in ids)
    if ctx1 - ctx0 != batch * steps:
        raise RuntimeError(f"decode batch {batch}: {ctx1 - ctx0} tokens decoded in {steps} steps")
    replays = runner.graphs.replays if runner.graphs is not None else 0
    check = check_decode_logits(runner, eng, ids, batch, alone)
    if runner.graphs is not None:
        if runner.graphs.replays <= replays:
            raise RuntimeError(f"decode batch {batch}: the checked step did not go through a recorded graph")
        log(f"  graphs: {runner.graphs.captures} captured, {runner.graphs.replays} replays so far")
    return batch * steps / dt, dt / steps, (ctx0 + ctx1) / 2, check


def sane_logits(rows, what):
    """The reference's rule for a run that computed nothing: all-zero logits fail
    (tests/test_gpu_identity.c:190-201); so do logits that are not finite, and rows that are constant."""
    import torch
    if not bool(torch.isfinite(rows).all()):
        raise RuntimeError(f"{what}: logits are not finite")
    if bool((rows.abs().amax(dim=-1) == 0).any()) or bool((rows.std(dim=-1) == 0).any()):
        raise RuntimeError(f"{what}: a row of logits is all zero or all equal")


def check_decode_logits(runner, eng, ids, batch, alone):
    """One more decode step of the timed batch, through the same recorded graph, with its logits
    looked at: every row finite, not zero, not constant.  With ``alone``, the first request's row is
    also compared with the same tokens run as a request of its own (its prompt in portions of 2,048,
    the last token as a decode step of one): (max, mean) difference as fractions of the mean logit
    range.  Ends the requests."""
    import torch
    from xyntetik_runner_amd.engine.batch import StepEntry
    eng.run_ahead = False
    eng.step()                       # the step that was queued ahead, if any: now the host knows every token
    reqs = [eng.requests[i] for i in ids]
    if any(r.remaining != 1 for r in reqs):
        raise RuntimeError(f"decode batch {batch}: a request is not decoding")
    logits = runner.step([StepEntry(r.id, [r.output[-1]], [0]) for r in reqs])
    sane_logits(logits, f"decode batch {batch}")
    row = logits[0].clone()
    tokens = list(reqs[0].prompt) + list(reqs[0].output)
    for i in ids:
        eng.abort(i)
    if not alone:
        return None
    for a in range(0, len(tokens) - 1, 2048):
        runner.step([StepEntry("alone", tokens[a:min(a + 2048, len(tokens) - 1)], [])])
    single = runner.step([StepEntry("alone", tokens[-1:], [0])])[0]
    runner.finish("alone")
    sane_logits(single[None], f"decode batch {batch}, the first request alone")
    span = float((single.max() - single.min()))
    d = (row - single).abs()
    return {"max": round(float(d.max()) / span, 5), "mean": round(float(d.mean()) / span, 6),
            "same_top": bool(int(row.argmax()) == int(single.argmax()))}


def measure_mixed(runner, cfg, n_requests, steps_each, seed):
    """A scheduler workload: `n_requests` prompts of 128..2048 tokens admitted at once, `steps_each`
    tokens decoded for each, portions of prompts beside decoded tokens under a 2048-token budget.
    Returns (prompt tokens, decoded tokens, seconds, steps)."""
    import numpy as np
    import torch
    from xyntetik_runner_amd.engine import Engine
    from xyntetik_runner_amd.sampling import SamplingParams
    eng = Engine(runner, max_batched_tokens=2048, max_running=n_requests,
                 max_model_len=cfg["max_position_embeddings"], stop_ids=[])
    rng = np.random.default_rng(seed)
    lens = [int(n) for n in rng.integers(128, 2049, size=n_requests)]
    sp = SamplingParams(temperature=0.0, max_new_tokens=steps_each, ignore_eos=True)
    for n in lens:
        eng.add_request([int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)], sp)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_steps = 0
    done = []
    while eng.has_work():
        done += [o.request for o in eng.step() if o.finished]
        n_steps += 1
    torch.cuda.synchronize()
    secs = time.perf_counter() - t0
    if len(done) != n_requests or any(len(r.output) != steps_each for r in done):
        raise RuntimeError("mixed workload: a request ended early")
    return sum(lens), n_requests * steps_each, secs, n_steps


def measure_prefill(runner, cfg, T, repeats, seed):
    import numpy as np
    import torch
    from xyntetik_runner_amd.engine.batch import StepEntry
    """Seconds for a prompt of T tokens in one step, up to the logits of its last position on the
    host: the median of ``repeats`` runs after one that is not counted (the reference reports
    medians, docs/benchmarks.md:16)."""
    rng = np.random.default_rng(seed)
    times = []
    for r in range(repeats + 1):
        toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=T)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = runner.step([StepEntry(("prefill", r), toks, [T - 1])])
        last = out.cpu()
        dt = time.perf_counter() - t0
        sane_logits(last, "prefill")
        runner.finish(("prefill", r))
        if r > 0:
            times.append(dt)
    times.sort()
    return times[len(times) // 2]


def measure_prefill_in_portions(runner, cfg, T, portion, seed):
    """Seconds for a prompt of T tokens run in portions of ``portion`` (each step reads the cache
    the portions before it left), up to the logits of its last position."""
    import numpy as np
    import torch
    from xyntetik_runner_amd.engine.batch import StepEntry
    rng = np.random.default_rng(seed)
    best = None
    for r in range(2):
        toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=T)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for a in range(0, T, portion):
            b = min(T, a + portion)
            out = runner.step([StepEntry(("long prefill", r), toks[a:b], [b - a - 1] if b == T else [])])
        out.cpu()
        dt = time.perf_counter() - t0
        runner.finish(("long prefill", r))
        best = dt if best is None else min(best, dt)
    return best


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="decode steps that are timed (the configuration decodes 256 tokens)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the configuration has (named in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--shape", default="llama-3.1-8b", choices=sorted(SHAPES), help="sizes of the model (same architecture)")
    ap.add_argument("--max-context", type=int, default=0, metavar="N",
                    help="the model's context length (max_position_embeddings) instead of the shape's own")
    ap.add_argument("--contexts", default="", metavar="LIST",
                    help="decode points at these context lengths (comma separated) instead of the points at the model's limit")
    ap.add_argument("--context-batches", default="1,8", metavar="LIST", help="batch sizes of the --contexts points")
    ap.add_argument("--long-prefill", type=int, default=0, metavar="T",
                    help="length of the prompt that is run in portions of 2,048 (default: the model's context)")
    ap.add_argument("--record", default="", metavar="FILE",
                    help="also write the command and the JSON line into FILE (markdown)")
    ap.add_argument("--mixed", type=int, default=0, metavar="N",
                    help="also run N requests with prompts of 128..2048 tokens and 128 decoded tokens each through the scheduler")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported by this engine", flush=True)
        return 2
    shape_name, shape_cfg = SHAPES[args.shape]
    cfg = {k: v for k, v in shape_cfg.items() if v is not None}
    layers_full = cfg["num_hidden_layers"]
    layers = args.layers or layers_full
    cfg["num_hidden_layers"] = layers
    if args.max_context:
        cfg["max_position_embeddings"] = args.max_context
    P, B = args.prompt_len, args.batch
    elt = 2 if args.dtype == "bfloat16" else 4
    ctx_max = cfg["max_position_embeddings"]
    long_steps, long_warmup = 32, 4
    span = P + args.warmup + args.steps + 80 + max(64, B)
    pool = max(max(64, B) * (-(-span // 64) * 64) + 4096, args.mixed * (2048 + 128 + 64))
    # The points away from the tuned one: (context, batch) pairs.  By default the model's limit at
    # batch 8 and, if the card has room for 64 requests of that length beside the weights, at batch 64.
    import torch
    kv_per_token = 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * layers * elt
    body, head = matmul_params(cfg, layers)
    weight_bytes = (body + (1 if cfg.get("tie_word_embeddings") else 2) * head) * elt
    total_mem = torch.cuda.get_device_properties(0).total_memory

    def pool_for(ctx, b):
        return b * (-(-(ctx + 128) // 64) * 64) + 4096
    if args.contexts:
        ctx_points = [(int(c), int(b)) for c in args.contexts.split(",") for b in args.context_batches.split(",")]
    else:
        ctx_points = [(ctx_max, 8), (ctx_max, 64)]
    left_out = [cb for cb in ctx_points if weight_bytes + pool_for(*cb) * kv_per_token >= 0.8 * total_mem or cb[0] > ctx_max]
    ctx_points = [cb for cb in ctx_points if cb not in left_out]
    long_T = args.long_prefill or min(ctx_max, 32768)
    if not args.no_points:
        pool = max([pool, long_T + 4096] + [pool_for(*cb) for cb in ctx_points])
    spec, runner = build_runner(cfg, args.dtype, max_tokens=pool, max_requests=max(64, args.mixed))

    read_gbs, mm_flops = measure_achievable(runner) if args.dtype == "bfloat16" else (None, None)
    if read_gbs:
        log(f"achievable on this GPU: {read_gbs:.0f} GB/s to a kernel that only reads, "
            f"{mm_flops / 1e12:.0f} TFLOP/s bfloat16 on a 8192 x 28672 x 4096 product")
    peak_flops = PEAK["bf16_flops" if args.dtype == "bfloat16" else "fp32_flops"]
    pre_s = measure_prefill(runner, cfg, 2048, repeats=5, seed=1)
    pre_rate = prefill_flops(cfg, layers, 2048) / pre_s
    log(f"prefill 2048 tokens: {pre_s * 1e3:.1f} ms (the median of 5)")

    # the decode figure: the median of three repetitions of the whole workload (fresh requests,
    # prompts computed again), as the reference reports a median of its runs
    # (docs/benchmarks.md:16)
    runs = []
    for rep in range(3):
        tps, step_s, ctx, _ = measure_decode(runner, cfg, B, P, args.steps, args.warmup, seed=2 + 100 * rep)
        runs.append((step_s, tps, ctx))
        log(f"decode batch {B}, repetition {rep + 1}: {tps:.1f} tok/s, {step_s * 1e3:.3f} ms/step, "
            f"{decode_bytes(cfg, layers, B, ctx, elt) / step_s / 1e9:.0f} GB/s")
    runs.sort()
    step_s, tps, ctx = runs[1]
    achieved = decode_bytes(cfg, layers, B, ctx, elt) / step_s / 1e9
    points, checks = {}, {}
    if not args.no_points:
        def point(name, b, prompt_len, n, warm, seed, alone=False):
            t, sec, c, chk = measure_decode(runner, cfg, b, prompt_len, n, warm, seed=seed, alone=alone)
            points[name] = round(t, 1)
            log(f"{name}: {t:.1f} tok/s, {sec * 1e3:.3f} ms/step, {decode_bytes(cfg, layers, b, c, elt) / sec / 1e9:.0f} GB/s")
            if chk is not None:
                # One request's logits must not depend on the 63 beside it beyond the rounding of bfloat16
                # operands summed in another order.  That rounding grows with the root of the depth:
                # measured on this shape against the engine's 32-bit path, bfloat16 differs by a mean of
                # 0.95e-3 of the logit range at 2 layers and 3.6e-3 at 32 (maximum 2.3e-2), a row in a
                # batch of 64 from the same row alone by 2.7e-3 (1.6e-2); a row computed from another
                # request's keys differs by its whole range.
                checks[f"{name}_row0_vs_alone"] = chk
                log(f"{name}: the first request's logits against the same request alone: {chk}")
                bound = 5e-3 * (max(layers, 2) / 32.0) ** 0.5
                if args.dtype == "bfloat16" and not (chk["mean"] <= bound and chk["max"] <= 10 * bound):
                    raise RuntimeError(f"{name}: a request's logits in the batch differ from the same request alone: {chk} "
                                       f"(allowed: mean {bound:.1e}, max {10 * bound:.1e} of the logit range)")
        for b in (1, 64):
            point(f"decode_b{b}", b, P, max(8, min(args.steps, 64)), min(args.warmup, 8), 3 + b, alone=b == 64)
        # away from the tuned point: long contexts (they end 128 tokens under the named length), and
        # a long prompt in portions
        for i, (c, b) in enumerate(ctx_points):
            # (the request admitted first decodes a token for every portion of the others' prompts;
            # it must not reach the model's limit before the last timed step)
            ahead = (b - 1) * -(-c // 2048) if c > 8192 else 0
            point(f"decode_b{b}_ctx{c}", b, c - 128 - ahead, long_steps if c <= 8192 else 16, long_warmup, 21 + i)
        for c, b in left_out:
            log(f"decode_b{b}_ctx{c}: left out, the cache of {b} such requests does not fit beside the weights "
                f"or the context is beyond the model's {ctx_max}")
        # short prompts (time to the first token's logits): steps of 128 and of 512 rows
        for T in (128, 512):
            short_s = measure_prefill(runner, cfg, T, repeats=5, seed=30 + T)
            points[f"prefill_{T}_tokens_ms"] = round(short_s * 1e3, 3)
            log(f"prefill {T} tokens: {short_s * 1e3:.2f} ms (the median of 5)")
        long_s = measure_prefill_in_portions(runner, cfg, long_T, 2048, seed=23)
        points[f"prefill_{long_T}_in_2048_portions"] = round(long_T / long_s, 1)
        log(f"prefill of {long_T} tokens in portions of 2048: {long_s * 1e3:.1f} ms, {long_T / long_s:.0f} tok/s")
    if args.mixed:
        # the workload twice: the first pass also records the decode graphs of its batch sizes (as the
        # warm-up steps do for the decode figures), the second is the figure; both are reported
        for name in ("mixed_first_pass_tok_s", "mixed_total_tok_s"):
            n_prompt, n_dec, secs, n_steps = measure_mixed(runner, cfg, args.mixed, 128, seed=9)
            log(f"mixed ({name}): {args.mixed} requests, {n_prompt} prompt + {n_dec} decoded tokens in {secs:.3f} s "
                f"({n_steps} steps): {(n_prompt + n_dec) / secs:.0f} tok/s in all, {n_dec / secs:.0f} decoded tok/s")
            points[name] = round((n_prompt + n_dec) / secs, 1)
    line = {
        "metric": f"decode tokens/s, {shape_name}, batch {B}, {P}-token prompts (random weights)",
        "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": shape_name, "layers": layers, "layers_in_config": layers_full,
                   "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
                   "global_batch": B, "seq_len": P, "max_context": cfg["max_position_embeddings"],
                   "decode_tokens": args.steps, "parallelism": "single GPU"},
        "prefill": {"value": round(2048 / pre_s, 1), "tokens": 2048, "ms": round(pre_s * 1e3, 3),
                    "frac": round(pre_rate / peak_flops, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK["hbm_gbs"], "unit": "GB/s",
                     "frac": round(achieved / PEAK["hbm_gbs"], 4)},
        "points": points, "checks": checks,
        "repetitions_ms_per_step": [round(r[0] * 1e3, 4) for r in runs],
    }
    if read_gbs:
        # the same two figures against what this GPU gave a kernel that only reads, and the matrix
        # kernel on one large product, in this very run
        line["roofline"]["measured_peak"] = round(read_gbs, 1)
        line["roofline"]["frac_of_measured"] = round(achieved / read_gbs, 4)
        # no roofline, and it can exceed 1: the step's rate over that of this engine's own matrix
        # kernel on one large product
        line["prefill"]["own_gemm_tflops"] = round(mm_flops / 1e12, 1)
        line["prefill"]["frac_of_own_gemm"] = round(pre_rate / mm_flops, 4)
    text = json.dumps(line)
    print(text, flush=True)
    if args.record:
        with open(args.record, "w") as f:
            f.write(f"# bench.py, {shape_name}\n\nCommand:\n\n    python {' '.join(['bench.py'] + sys.argv[1:])}\n\n"
                    f"Result (one MI355X, random weights, synthetic tokens):\n\n```json\n{json.dumps(line, indent=1)}\n```\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
