"""The command line, with the reference's option names and meanings where it has them
(src/main.c:188-340 usage, :505-639 parsing):

  -m PATH   model folder (config.json + model.safetensors; the reference takes a GGUF file)
  -p TEXT   prompt; \\n, \\t, \\\\ are unescaped; echoed before the completion (:509, :1519, :1541)
  -f FILE   prompt from a file, appended after -p
  -n N      tokens to generate, default 256, -1 = until a stop token (:511)
  -c N      context length (default: the model's, at most 4096) (:3075)
  -b N      tokens per prompt portion / step budget (default 512)
  -s N      seed of the sampler; 0 is refused (:833-845)
  --temp F  temperature, 0 = greedy (default 0)
  --top-k N / --top-p F / --min-p F / --repeat-penalty F   (:254-262)
  --ignore-eos, --no-bos, --bench-json, --version, -v, -h

and, for models that come without a tokenizer: --ids 1,2,3 gives the prompt as token
ids and prints ids.  Without --ids and without a tokenizer.json in the model folder the
prompt's bytes are the ids (byte b is token b).

stdout gets the prompt and the generated text and a newline; stderr gets
"[end of text]" when a stop token ended it, then
"prompt: N tok, X tok/s | gen: N tok, Y tok/s" (:1541-1549).
"""
from __future__ import annotations

import json
import os
import sys
import time
from typing import List, Optional

VERSION_LINE = "runner (xyntetik-runner_amd) {v}"

USAGE = """usage: runner -m MODEL_DIR [options]

options:
  -m PATH        the model: a folder holding config.json and model.safetensors
  -p TEXT        the prompt to complete; backslash escapes such as \\n are expanded
  -f FILE        take the prompt from FILE (it follows the -p text if both are given)
  --ids LIST     the prompt as token ids separated by commas; the answer is printed as ids too
  -n N           how many tokens to generate at most (default 256; -1: stop only at an end token)
  -c N           context length in tokens (default: the model's own limit, capped at 4096)
  -b N           how many prompt tokens one step may take (default 512)
  -s N           seed of the sampler's generator (default: from the clock; 0 is refused)
  --temp F       sampling temperature (default 0 = always the most likely token,
                 and then no repeat penalty either)
  --top-k N      sample among the N most likely tokens only (0: no limit)
  --top-p F      sample from the smallest set of tokens whose probabilities reach F
  --min-p F      drop tokens less likely than F times the most likely one (0: keep all)
  --repeat-penalty F  make tokens of the recent window less likely by factor F (1: off)
  --no-bos       do not put the begin-of-sequence token before the prompt
  --ignore-eos   go on generating when an end token comes
  --dtype T      bfloat16 (default) or float32
  --bench-json   time a short generation and print the figures as JSON
  --version      print the version and leave
  -v             print the model's sizes while loading
"""


class UsageError(Exception):
    pass


def unescape(s: str) -> str:
    out, i = [], 0
    while i < len(s):
        if s[i] == "\\" and i + 1 < len(s):
            c = s[i + 1]
            out.append({"n": "\n", "t": "\t", "r": "\r", "\\": "\\", '"': '"'}.get(c, "\\" + c))
            i += 2
        else:
            out.append(s[i])
            i += 1
    return "".join(out)


def parse_args(argv: List[str]) -> dict:
    o = dict(model=None, prompt=None, file=None, ids=None, n=256, ctx=0, batch=512, seed=None, temp=0.0,
             top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, no_bos=False, ignore_eos=False,
             dtype="bfloat16", bench_json=False, version=False, verbose=False, help=False)
    i = 0

    def val(flag):
        nonlocal i
        if i + 1 >= len(argv):
            raise UsageError(f"option {flag} needs a value")
        i += 1
        return argv[i]

    def num(flag, conv):
        v = val(flag)
        try:
            return conv(v)
        except ValueError:
            raise UsageError(f"option {flag}: {v!r} is not a number") from None

    while i < len(argv):
        a = argv[i]
        if a == "-m": o["model"] = val(a)
        elif a == "-p": o["prompt"] = val(a)
        elif a == "-f": o["file"] = val(a)
        elif a == "--ids": o["ids"] = val(a)
        elif a == "-n": o["n"] = num(a, int)
        elif a == "-c": o["ctx"] = num(a, int)
        elif a == "-b": o["batch"] = num(a, int)
        elif a == "-s": o["seed"] = num(a, int)
        elif a == "--temp": o["temp"] = num(a, float)
        elif a == "--top-k": o["top_k"] = num(a, int)
        elif a == "--top-p": o["top_p"] = num(a, float)
        elif a == "--min-p": o["min_p"] = num(a, float)
        elif a == "--repeat-penalty": o["repeat_penalty"] = num(a, float)
        elif a == "--no-bos": o["no_bos"] = True
        elif a == "--ignore-eos": o["ignore_eos"] = True
        elif a == "--dtype": o["dtype"] = val(a)
        elif a == "--bench-json": o["bench_json"] = True
        elif a == "--version": o["version"] = True
        elif a == "-v": o["verbose"] = True
        elif a in ("-h", "--help"): o["help"] = True
        else:
            raise UsageError(f"unknown option {a}")
        i += 1
    return o


class Tokens:
    """Text <-> ids: tokenizer.json if the folder has one, else bytes as ids."""

    def __init__(self, model_dir: str, vocab: int):
        self.tk = None
        path = os.path.join(model_dir, "tokenizer.json")
        if os.path.exists(path):
            from tokenizers import Tokenizer
            self.tk = Tokenizer.from_file(path)
        self.vocab = vocab

    def encode(self, text: str) -> List[int]:
        if self.tk is not None:
            return list(self.tk.encode(text, add_special_tokens=False).ids)
        ids = list(text.encode("utf-8"))
        if ids and max(ids) >= self.vocab:
            raise UsageError(f"the prompt's bytes do not fit a vocabulary of {self.vocab}; give --ids")
        return ids

    def decode(self, ids: List[int]) -> str:
        if self.tk is not None:
            return self.tk.decode(ids, skip_special_tokens=False)
        return bytes(i for i in ids if i < 256).decode("utf-8", "replace")


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    try:
        o = parse_args(argv)
    except UsageError as e:
        sys.stderr.write(f"error: {e}\n{USAGE}")
        return 1
    if o["help"]:
        sys.stderr.write(USAGE)
        return 0
    if o["version"]:
        from . import __version__
        print(VERSION_LINE.format(v=__version__))
        return 0
    if not o["model"]:
        sys.stderr.write(USAGE)
        return 1
    if o["seed"] is not None and o["seed"] == 0:
        sys.stderr.write("error: seed 0 cannot be used (-s 0): the sampler's generator never leaves state 0. "
                         "Any other seed will do.\n")
        return 1
    from .config import ConfigError, load_config
    from .weights import SafetensorsError, WeightError
    try:
        arch, cfg = load_config(o["model"])
    except ConfigError as e:
        sys.stderr.write(f"error: {e}\n")
        return 1
    spec = arch.build_spec(cfg)
    if o["verbose"]:
        sys.stderr.write(f"model: {spec.architecture}, {len(spec.layers)} layers, width {spec.hidden_size}, "
                         f"vocabulary {spec.vocab_size}, context {spec.max_position}\n")
    ctx = o["ctx"] if o["ctx"] > 0 else min(spec.max_position, 4096)

    toks = Tokens(o["model"], spec.vocab_size)
    text = ""
    if o["prompt"] is not None:
        text += unescape(o["prompt"])
    if o["file"] is not None:
        try:
            with open(o["file"], "r", encoding="utf-8") as f:
                text += f.read()
        except OSError as e:
            sys.stderr.write(f"error: cannot read {o['file']}: {e}\n")
            return 1
    try:
        if o["ids"] is not None:
            prompt = [int(t) for t in o["ids"].replace(" ", "").split(",") if t != ""]
        elif o["bench_json"] and not text:
            prompt = [(7919 + i * 104729) % spec.vocab_size for i in range(min(512, ctx // 2))]
        else:
            if not text:
                sys.stderr.write("error: no prompt (give -p, -f or --ids)\n")
                return 1
            prompt = toks.encode(text)
            if spec.bos_token_id is not None and not o["no_bos"]:
                prompt = [spec.bos_token_id] + prompt
    except (UsageError, ValueError) as e:
        sys.stderr.write(f"error: {e}\n")
        return 1
    if not prompt:
        sys.stderr.write("error: the prompt is empty\n")
        return 1
    if len(prompt) >= ctx:
        sys.stderr.write(f"error: the prompt has {len(prompt)} tokens and does not fit a context of {ctx}; "
                         f"-c {len(prompt) + max(o['n'], 1)} would\n")
        return 1

    from .engine import Engine, ModelRunner
    from .sampling import SamplingParams
    try:
        runner = ModelRunner.from_folder(o["model"], dtype=o["dtype"], max_tokens=ctx, page_size=64, max_requests=1)
    except (WeightError, SafetensorsError, ValueError) as e:
        sys.stderr.write(f"error: {e}\n")
        return 1
    engine = Engine(runner, max_batched_tokens=max(1, o["batch"]), max_running=1, max_model_len=ctx)
    params = SamplingParams(temperature=o["temp"], top_k=o["top_k"], top_p=o["top_p"], min_p=o["min_p"],
                            repeat_penalty=o["repeat_penalty"], seed=o["seed"], max_new_tokens=o["n"],
                            ignore_eos=o["ignore_eos"] or o["bench_json"])
    import torch
    as_ids = o["ids"] is not None
    if not o["bench_json"]:
        sys.stdout.write(",".join(map(str, prompt)) if as_ids else text)
        sys.stdout.flush()
    rid = engine.add_request(prompt, params)
    req = engine.requests[rid]          # (the engine drops it when it ends; its last output brings it again)
    t0 = time.perf_counter()
    t_first = None
    n_gen = 0
    while engine.has_work():
        for out in engine.step():
            if out.token is not None:
                if t_first is None:
                    torch.cuda.synchronize()
                    t_first = time.perf_counter()
                n_gen += 1
                if not o["bench_json"]:
                    sys.stdout.write(("," + str(out.token)) if as_ids else toks.decode([out.token]))
                    sys.stdout.flush()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    prompt_s = (t_first or t1) - t0
    gen_s = max(t1 - (t_first or t1), 1e-9)
    p_rate = len(prompt) / max(prompt_s, 1e-9)
    g_rate = max(n_gen - 1, 0) / gen_s if n_gen > 1 else 0.0
    if o["bench_json"]:
        print(json.dumps({"prompt_tokens": len(prompt), "prompt_s": prompt_s, "prompt_tok_s": p_rate,
                          "gen_tokens": n_gen, "gen_s": gen_s, "gen_tok_s": g_rate, "dtype": o["dtype"]}))
        return 0
    sys.stdout.write("\n")
    if req.finish_reason == "stop":
        sys.stderr.write("[end of text]\n")
    sys.stderr.write(f"prompt: {len(prompt)} tok, {p_rate:.1f} tok/s | gen: {n_gen} tok, {g_rate:.1f} tok/s\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
