"""The command line, in the manner of the reference's `denno` (crates/denno-cli/src/main.rs:19-102):

    denno generate <model> --prompt TEXT [--system TEXT] [--max-tokens 128] [--temperature T]
          [--seed N] [--repetition-penalty P] [--frequency-penalty F] [--presence-penalty P]
          [--no-repeat-ngram-size N] [--quant fp32|bf16] [--raw]
    denno info <model>
    denno random-model <folder> --config FILE --seed N [--dtype float32|bfloat16]

    denno generate <model> --prompt-file FILE [--max-live N] [--page-size N] [--cache-tokens N]
          [--prefill-chunk N] [--max-batch-tokens N] [--kv-policy preempt|reserve] ...

`<model>` is a folder with config.json and model.safetensors (the reference resolves a hub id
in its download cache, main.rs:555-565; there is no network here).  Option names and defaults
are the reference's: max-tokens 128, temperature unset = 1.0 and 0 = greedy, seed unset =
entropy.  `--quant` names the precision: the reference's fp32 (default there) and this
engine's bf16; its int8 and q4 modes are not built.  Beyond the reference: `--prompt-ids`
for token ids where the folder has no tokenizer.json, `--top-k`, `--top-p`, `--stop` (the reference's
request parameters, crates/denno-engine/src/engine.rs:42-44), `--ignore-eos`; `--prompt-file` with
one prompt a line (token ids separated by commas or blanks), which all go through the scheduler
together, one line of output each in the file's order; and the engine's own options (`--max-live`,
`--page-size`, `--cache-tokens`, `--prefill-chunk`, `--max-batch-tokens`, `--kv-policy`,
`--no-graphs`), which the reference sets through DENNO_* environment variables.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def fallback_template(system, prompt):
    """The reference's template for models without one: 'system: ..\\n\\nuser: ..\\n\\nassistant:'
    (crates/denno-engine/src/tokenizer.rs:226-236)."""
    s = ""
    if system:
        s += f"system: {system}\n\n"
    s += f"user: {prompt}\n\n"
    return s + "assistant:"


def load_tokenizer(model_dir):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(path)


def parser():
    ap = argparse.ArgumentParser(prog="denno", description="inference engine for one MI355X")
    sub = ap.add_subparsers(dest="command", required=True)
    g = sub.add_parser("generate", help="one generation")
    g.add_argument("model", help="model folder")
    g.add_argument("--prompt", help="prompt text (needs tokenizer.json in the folder)")
    g.add_argument("--prompt-ids", help="prompt as comma-separated token ids")
    g.add_argument("--prompt-file", help="several prompts, one a line, as token ids separated by commas or blanks")
    g.add_argument("--system", default=None)
    g.add_argument("--max-tokens", type=int, default=128)
    g.add_argument("--temperature", type=float, default=None, help="unset: 1.0; 0: greedy")
    g.add_argument("--top-k", type=int, default=None)
    g.add_argument("--top-p", type=float, default=None)
    g.add_argument("--seed", type=int, default=None)
    g.add_argument("--stop", action="append", default=None,
                   help="a text that ends the generation where it first appears (needs tokenizer.json); may be given more than once")
    g.add_argument("--repetition-penalty", type=float, default=None)
    g.add_argument("--frequency-penalty", type=float, default=None)
    g.add_argument("--presence-penalty", type=float, default=None)
    g.add_argument("--no-repeat-ngram-size", type=int, default=None)
    g.add_argument("--quant", default="bf16", help="fp32 | bf16")
    g.add_argument("--raw", action="store_true", help="no chat template")
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--cast-weights", action="store_true",
                   help="bf16: round matrices stored in 32-bit to bfloat16 at load")
    g.add_argument("--max-live", type=int, default=None,
                   help="most requests that hold cache at a time (default: 1, or up to 64 with --prompt-file)")
    g.add_argument("--page-size", type=int, default=16, help="tokens in a page of the cache")
    g.add_argument("--cache-tokens", type=int, default=None,
                   help="size of the cache in tokens (default: max-live times the model's positions)")
    g.add_argument("--prefill-chunk", type=int, default=512, help="longest portion of one prompt in one step")
    g.add_argument("--max-batch-tokens", type=int, default=2048, help="token budget of one step")
    g.add_argument("--kv-policy", default="preempt", choices=["preempt", "reserve"],
                   help="when pages run out: preempt the youngest request, or admit only what can be reserved")
    g.add_argument("--no-graphs", action="store_true", help="run decode steps kernel by kernel")
    i = sub.add_parser("info", help="what a model folder holds")
    i.add_argument("model")
    r = sub.add_parser("random-model", help="write a model folder with random weights")
    r.add_argument("folder")
    r.add_argument("--config", required=True, help="a config.json to take sizes from")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", default="float32", choices=["float32", "bfloat16"])
    return ap


def cmd_generate(a):
    from .config import EngineOptions
    from .engine import Engine, SamplingParams
    quant = {"fp32": "float32", "float32": "float32", "bf16": "bfloat16", "bfloat16": "bfloat16"}.get(a.quant)
    if quant is None:
        raise SystemExit(f"--quant {a.quant}: this engine has fp32 and bf16; quantized weights are not built")
    tok = load_tokenizer(a.model)
    if a.prompt_file is not None:
        with open(a.prompt_file) as f:
            prompts = [[int(x) for x in line.replace(",", " ").split()] for line in f if line.strip()]
        if not prompts:
            raise SystemExit(f"{a.prompt_file} holds no prompt")
    elif a.prompt_ids is not None:
        ids = [int(x) for x in a.prompt_ids.replace(" ", "").split(",") if x]
    elif a.prompt is not None:
        if tok is None:
            raise SystemExit(f"{a.model} has no tokenizer.json (or the tokenizers package is missing): "
                             "give the prompt as --prompt-ids")
        text = a.prompt if a.raw else fallback_template(a.system, a.prompt)
        ids = tok.encode(text).ids
    else:
        raise SystemExit("one of --prompt, --prompt-ids and --prompt-file is needed")
    if a.prompt_file is None:
        prompts = [ids]
    params = SamplingParams(
        max_tokens=a.max_tokens, temperature=a.temperature, top_k=a.top_k, top_p=a.top_p, seed=a.seed,
        repetition_penalty=a.repetition_penalty, frequency_penalty=a.frequency_penalty,
        presence_penalty=a.presence_penalty, no_repeat_ngram_size=a.no_repeat_ngram_size,
        ignore_eos=a.ignore_eos, stop_sequences=tuple(a.stop or ()))
    if a.stop and tok is None:
        raise SystemExit(f"--stop is a text: {a.model} has no tokenizer.json (or the tokenizers package is missing)")
    max_live = a.max_live if a.max_live is not None else min(len(prompts), 64)
    eng = Engine.from_folder(a.model, EngineOptions(
        dtype=quant, max_live=max_live, seed=a.seed, page_size=a.page_size, cache_tokens=a.cache_tokens,
        prefill_chunk=a.prefill_chunk, max_batch_tokens=a.max_batch_tokens, kv_policy=a.kv_policy,
        use_graphs=not a.no_graphs), a.cast_weights,
        detokenize=(lambda ids: tok.decode(list(ids))) if tok is not None else None)
    for rid, out in enumerate(eng.generate(prompts, params)):
        if a.raw or tok is None:
            # the raw path stops at the end-of-sequence token without keeping it (main.rs:708-710)
            eos = set(eng.spec.eos_token_ids)
            if out and out[-1] in eos and not a.ignore_eos:
                out = out[:-1]
        if tok is not None and a.prompt is not None:
            text = eng.requests[rid].text      # cut at a stop sequence, where one ended it
            print(text if text is not None else tok.decode(out))
        else:
            print(",".join(str(t) for t in out))
    return 0


def cmd_info(a):
    from .config import load_config
    from .weights import open_checkpoint
    arch, cfg = load_config(a.model)
    where, files = open_checkpoint(a.model)
    n = sum(1 for _ in where)
    params = 0
    dtypes = {}
    for name, sf in where.items():
        dt, shape = sf.entries[name]
        k = 1
        for s in shape:
            k *= s
        params += k
        dtypes[dt] = dtypes.get(dt, 0) + 1
    for f in files:
        f.close()
    print(json.dumps({"architecture": arch.name, "config": cfg.to_dict(), "tensors": n, "parameters": params,
                      "stored": dtypes}, indent=1))
    return 0


def cmd_random_model(a):
    from .weights import write_model_folder
    with open(a.config) as f:
        cfg = json.load(f)
    write_model_folder(a.folder, cfg, a.seed, a.dtype)
    print(a.folder)
    return 0


def main(argv=None):
    a = parser().parse_args(argv)
    return {"generate": cmd_generate, "info": cmd_info, "random-model": cmd_random_model}[a.command](a)


if __name__ == "__main__":
    sys.exit(main())
