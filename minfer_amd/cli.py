"""Command line in the manner of the reference's (`src/main.rs:72-118,147-291` of
yusiwen/minfer): a hand-rolled flag loop, the same option names, meanings and defaults where
the reference has them, usage plus exit status 1 for an unknown flag or a missing or
unparsable value.  Prompts are token ids (there is no tokenizer here).

    minfer <model_dir> --prompt-tokens 1,2,3 [OPTIONS]
    minfer --config config.json --random-weights --prompt-tokens "1,2,3;4,5" [OPTIONS]
"""
from __future__ import annotations

import sys
from typing import List, Optional

USAGE = """minfer_amd - a minimal LLM inference engine for AMD MI355X

USAGE:
  {prog} <model_dir> --prompt-tokens <IDS> [OPTIONS]
  {prog} --config <config.json> --random-weights --prompt-tokens <IDS> [OPTIONS]

MODEL - <model_dir> is a folder with config.json and model.safetensors.

OPTIONS:
  --prompt-tokens <IDS>   token ids, comma separated; ';' separates the prompts of a
                          batch; @FILE reads them from a file (one prompt a line)
  --random-weights        random weights from the configuration and --weight-seed
  --config <FILE>         config.json to use with --random-weights
  --weight-seed <N>       seed of the random weights (default 0)
  --dtype <T>             bfloat16 (default) or float32
  --temp <T>              temperature of the draw; below 1e-6 the largest logit is taken
                          (default 0.8)
  --greedy                the same as --temp 0
  --top-k <K>             draw among the K largest logits only; 0 keeps all (default 40)
  --top-p <P>             draw among the most probable tokens that together reach P; values
                          outside (0, 1) keep all (default 0.95)
  --repeat-penalty <N>    logits of the last 64 tokens are divided by N (multiplied if
                          negative); 1.0 leaves them (default 1.1)
  --frequency-penalty <N> N times a token's count among the last 64 is taken off its logit
                          (default 0.0)
  --presence-penalty <N>  N is taken off the logit of every token among the last 64
                          (default 0.0)
  --stop-token <ID>       a token id that ends a sequence and is not emitted; may be given
                          several times (default: the model's eos ids)
  -n, --n-predict <N>     most tokens generated per prompt (default 512); also --max-new
  --seed <N>              seed of the sampler's random streams (default 42)
  --n-ctx <N>             context per sequence (default 4096)
  --n-slots <N>           sequences decoded together (default: number of prompts, at most 64)
  --no-graph              do not capture the decode step as a HIP graph
  -h, --help              show this help
  -V, --version           print version and exit
"""


class UsageError(Exception):
    pass


def parse_prompts(text: str) -> List[List[int]]:
    if text.startswith("@"):
        with open(text[1:]) as f:
            chunks = [l.strip() for l in f if l.strip()]
    else:
        chunks = [c for c in text.split(";") if c.strip()]
    prompts = []
    for c in chunks:
        try:
            prompts.append([int(t) for t in c.replace(",", " ").split()])
        except ValueError:
            raise UsageError(f"--prompt-tokens: not a list of token ids: {c!r}") from None
    if not prompts or any(not p for p in prompts):
        raise UsageError("--prompt-tokens: no tokens")
    return prompts


def parse_args(argv: List[str]) -> dict:
    o = dict(model=None, prompt_tokens=None, random_weights=False, config=None, weight_seed=0,
             dtype="bfloat16", temp=0.8, top_k=40, top_p=0.95, repeat_penalty=1.1, frequency_penalty=0.0,
             presence_penalty=0.0, stop_tokens=None, n_predict=512, seed=42, n_ctx=4096, n_slots=None,
             graph=True, help=False, version=False)
    valued = {
        "--prompt-tokens": ("prompt_tokens", str), "--config": ("config", str),
        "--weight-seed": ("weight_seed", int), "--dtype": ("dtype", str), "--temp": ("temp", float),
        "-t": ("temp", float), "--top-k": ("top_k", int), "--top-p": ("top_p", float),
        "--repeat-penalty": ("repeat_penalty", float), "--frequency-penalty": ("frequency_penalty", float),
        "--presence-penalty": ("presence_penalty", float), "-n": ("n_predict", int),
        "--n-predict": ("n_predict", int), "--max-new": ("n_predict", int), "--seed": ("seed", int),
        "--n-ctx": ("n_ctx", int), "--n-slots": ("n_slots", int)}
    i = 0
    while i < len(argv):
        a = argv[i]
        if a in ("-h", "--help"):
            o["help"] = True
        elif a in ("-V", "--version"):
            o["version"] = True
        elif a == "--greedy":
            o["temp"] = 0.0
        elif a == "--random-weights":
            o["random_weights"] = True
        elif a == "--no-graph":
            o["graph"] = False
        elif a == "--stop-token" or a in valued:
            if i + 1 >= len(argv):
                raise UsageError(f"{a} requires a value")
            raw = argv[i + 1]
            i += 1
            try:
                if a == "--stop-token":
                    o["stop_tokens"] = (o["stop_tokens"] or []) + [int(raw)]
                else:
                    key, conv = valued[a]
                    o[key] = conv(raw)
            except ValueError:
                raise UsageError(f"{a}: cannot parse {raw!r}") from None
        elif a.startswith("-") and len(a) > 1:
            raise UsageError(f"unknown option {a}")
        elif o["model"] is None:
            o["model"] = a
        else:
            raise UsageError(f"unexpected argument {a!r} (prompts are given with --prompt-tokens)")
        i += 1
    return o


def main(argv: Optional[List[str]] = None, prog: str = "minfer") -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    try:
        o = parse_args(argv)
        if o["help"]:
            print(USAGE.format(prog=prog), file=sys.stderr)
            return 0
        if o["version"]:
            from . import __version__
            print(f"minfer_amd {__version__}")
            return 0
        if o["dtype"] not in ("bfloat16", "bf16", "float32", "fp32"):
            raise UsageError(f"--dtype: {o['dtype']!r} is not bfloat16 or float32")
        if o["prompt_tokens"] is None:
            raise UsageError("--prompt-tokens is required")
        if o["model"] is None and not (o["random_weights"] and o["config"]):
            raise UsageError("a model folder is required (or --config with --random-weights)")
        prompts = parse_prompts(o["prompt_tokens"])
    except UsageError as e:
        print(f"Error: {e}\n", file=sys.stderr)
        print(USAGE.format(prog=prog), file=sys.stderr)
        return 1

    from .api import LLM
    from .config.base import ConfigError
    from .weights.loader import WeightError
    n_slots = o["n_slots"] or min(len(prompts), 64)
    try:
        llm = LLM(o["model"], config=o["config"], random_weights=o["random_weights"],
                  weight_seed=o["weight_seed"], dtype=o["dtype"], n_ctx=o["n_ctx"], n_slots=n_slots)
        res = llm.generate(prompts, max_new=o["n_predict"], temp=o["temp"], top_k=o["top_k"], top_p=o["top_p"],
                           repeat_penalty=o["repeat_penalty"], frequency_penalty=o["frequency_penalty"],
                           presence_penalty=o["presence_penalty"], seed=o["seed"],
                           stop_tokens=o["stop_tokens"], use_graph=o["graph"])
    except (ConfigError, WeightError, ValueError, RuntimeError) as e:
        print(f"Error: {e}", file=sys.stderr)
        return 1
    for toks in res.tokens:
        print(",".join(str(t) for t in toks))
    n_gen = sum(len(t) for t in res.tokens)
    total_s = res.prefill_seconds + res.decode_seconds
    print(f"\nPrefill: {res.prefill_tokens} tokens in {res.prefill_seconds:.3f} s "
          f"({res.prefill_rate:.1f} tok/s)", file=sys.stderr)
    print(f"Generated: {n_gen} tokens in {res.decode_seconds:.3f} s ({res.decode_rate:.1f} tok/s)",
          file=sys.stderr)
    print(f"Total: {res.prefill_tokens + n_gen} tokens in {total_s:.3f} s "
          f"({(res.prefill_tokens + n_gen) / total_s if total_s > 0 else 0.0:.1f} tok/s)", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
