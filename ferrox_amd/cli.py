"""Command line in the manner of the reference's `ferrox -m ... -p ... -n ...`
(ferrox-cli/src/run.rs:19-125, main.rs:254-296): the same flag names and
defaults where this engine has the feature.  The model is a folder with
config.json and safetensors, not a GGUF file; or, with --random-weights, a
configuration alone (--config FILE, or the name of one of the shapes that
`ferrox_amd.config.presets` holds) whose weights are drawn from --seed, as the
reference serves synthetic weights when it is given no model
(ferrox-server/src/model.rs:228-243).  The prompt is text when the folder holds
a tokenizer.json (or --tokenizer names one; read with the `tokenizers`
package), else token ids through --tokens.  Generated text (or ids) goes to
stdout, timings to stderr (run.rs:680-695).
"""
from __future__ import annotations

import argparse
import os
import sys
import time

from .config import presets


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="ferrox-amd", description="Qwen2-MoE text generation on one MI355X")
    ap.add_argument("-m", "--model", metavar="DIR", help="model folder (config.json + safetensors)")
    ap.add_argument("--random-weights", action="store_true",
                    help="no model folder: weights drawn from --seed for the configuration that --config names")
    ap.add_argument("--config", metavar="FILE|NAME", default="qwen1.5-moe-a2.7b",
                    help="with --random-weights: a config.json, or one of: " + ", ".join(presets.names()))
    ap.add_argument("--layers", type=int, default=0, help="with --random-weights: build only so many layers (0 = all)")
    ap.add_argument("--tokenizer", metavar="FILE", help="tokenizer.json (default: the one in the model folder)")
    ap.add_argument("-p", "--prompt", default="", help="prompt text (needs tokenizer.json in the model folder)")
    ap.add_argument("-f", "--file", metavar="FILE", help="read the prompt from a file")
    ap.add_argument("--tokens", metavar="IDS", help="prompt as comma-separated token ids")
    ap.add_argument("-n", "--n-predict", type=int, default=128, help="tokens to predict (-1 = fill the context)")
    ap.add_argument("-c", "--ctx-size", type=int, default=0, help="context size (0 = the model's)")
    ap.add_argument("-t", "--threads", type=int, default=0, help="accepted for compatibility; the GPU does the work")
    ap.add_argument("--temp", type=float, default=0.8, dest="temperature", help="sampling temperature (0 = greedy)")
    ap.add_argument("--top-k", type=int, default=40, help="top-k sampling (0 = off)")
    ap.add_argument("--top-p", type=float, default=0.95, help="nucleus sampling (1.0 = off)")
    ap.add_argument("--repeat-penalty", type=float, default=1.1, help="repetition penalty (1.0 = off)")
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("-s", "--seed", type=int, default=-1, help="RNG seed (-1 = from the clock)")
    ap.add_argument("--ignore-eos", action="store_true", help="ignore EOS and always emit -n tokens")
    ap.add_argument("--no-cnv", action="store_true", help="raw prompt (no chat template is ever applied here)")
    ap.add_argument("-e", "--escape", action="store_true", help="process \\n \\t \\r \\\\ escapes in -p")
    ap.add_argument("--verbose-prompt", action="store_true", help="print the prompt's token ids first")
    ap.add_argument("-dev", "--device", default="cuda:0")
    # engine knobs
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "bfloat16", "fp32", "float32"])
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--num-pages", type=int, default=0, help="cache pages per layer group (0 = from the context)")
    ap.add_argument("--max-tokens-per-step", type=int, default=4096)
    ap.add_argument("--prefill-chunk", type=int, default=4096,
                    help="most tokens of one prompt in a step (a step streams every expert it uses once, so large portions pay)")
    return ap


def unescape(s: str) -> str:
    out, i = [], 0
    table = {"n": "\n", "t": "\t", "r": "\r", "\\": "\\"}
    while i < len(s):
        if s[i] == "\\" and i + 1 < len(s) and s[i + 1] in table:
            out.append(table[s[i + 1]])
            i += 2
        else:
            out.append(s[i])
            i += 1
    return "".join(out)


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if bool(args.model) == bool(args.random_weights):
        print("error: give either a model folder (-m DIR) or --random-weights [--config FILE|NAME]", file=sys.stderr)
        return 2
    tokenizer = None
    tok_path = args.tokenizer or (os.path.join(args.model, "tokenizer.json") if args.model else "")
    if args.tokenizer and not os.path.isfile(tok_path):
        print(f"error: no tokenizer file at {tok_path}", file=sys.stderr)
        return 2
    if tok_path and os.path.isfile(tok_path):
        try:
            from tokenizers import Tokenizer
            tokenizer = Tokenizer.from_file(tok_path)
        except Exception as e:  # a broken tokenizer file is not fatal when --tokens is used
            print(f"warning: tokenizer.json could not be read ({e})", file=sys.stderr)
    if args.tokens:
        try:
            prompt_ids = [int(x) for x in args.tokens.replace(" ", "").split(",") if x]
        except ValueError:
            print("error: --tokens wants comma-separated integers", file=sys.stderr)
            return 2
    else:
        text = args.prompt
        if args.file:
            with open(args.file) as f:
                text = f.read()
        if args.escape:
            text = unescape(text)
        if tokenizer is None:
            print("error: no tokenizer.json (in the model folder or through --tokenizer); give the prompt as --tokens 1,2,3",
                  file=sys.stderr)
            return 2
        prompt_ids = tokenizer.encode(text).ids
    if not prompt_ids:
        print("error: empty prompt", file=sys.stderr)
        return 2
    if args.verbose_prompt:
        print("prompt tokens:", prompt_ids, file=sys.stderr)

    import torch
    if not torch.cuda.is_available():
        print("error: no GPU is visible; this engine has no CPU path", file=sys.stderr)
        return 2
    from .csrc.build import KernelBuildError
    from .engine.api import Engine
    from .sampling.sampler import SamplingParams

    # everything that can be wrong with the folder, the configuration, the weights or the request ends the
    # program with one message and exit code 2 (the reference bails the same way, run.rs:598-607)
    try:
        t0 = time.time()
        seed = args.seed if args.seed >= 0 else (time.time_ns() & 0x7FFFFFFFFFFFFFFF)       # run.rs:462-471
        source = dict(model_dir=args.model)
        if args.random_weights:
            from .config.base import read_config_json
            raw = read_config_json(args.config) if os.path.exists(args.config) else presets.load(args.config)
            if args.layers > 0:
                raw = dict(raw, num_hidden_layers=args.layers)
            source = dict(config=raw, random_weights=seed)
            print(f"random weights: seed {seed}, configuration {args.config}", file=sys.stderr)
        engine = Engine(**source, dtype=args.dtype, device=args.device, block_size=args.block_size,
                        num_pages=args.num_pages or None, max_seqs=4, ctx_size=args.ctx_size,
                        max_tokens_per_step=args.max_tokens_per_step, prefill_chunk=args.prefill_chunk)
        print(f"load time: {time.time() - t0:.2f} s", file=sys.stderr)
        defaulted = getattr(getattr(engine.model, "config", None), "defaulted_keys", ())
        if defaulted:                                                                    # run.rs:520-528
            print("config keys defaulted: " + ", ".join(defaulted), file=sys.stderr)
        params = SamplingParams(args.temperature, args.top_k, args.top_p, args.repeat_penalty,
                                args.presence_penalty, args.frequency_penalty, seed)
        t1 = time.time()
        shown = {"ids": [], "text": ""}

        def show(_, token):                 # printed as it is generated (run.rs:651-676)
            shown["ids"].append(token)
            if tokenizer is None:
                sys.stdout.write(("," if len(shown["ids"]) > 1 else "") + str(token))
            else:
                text = tokenizer.decode(shown["ids"])
                if text.endswith("\ufffd"):        # half of a character: wait for the rest
                    return
                sys.stdout.write(text[len(shown["text"]):])
                shown["text"] = text
            sys.stdout.flush()

        out = engine.generate_detailed([prompt_ids], args.n_predict, params, ignore_eos=args.ignore_eos, on_token=show)[0]
    except (ValueError, OSError, KernelBuildError) as e:     # ConfigError, CheckpointError, SafetensorsError are ValueErrors
        print(f"error: {e}", file=sys.stderr)
        return 2
    dt = time.time() - t1
    if tokenizer is not None:
        print(tokenizer.decode(out.token_ids)[len(shown["text"]):])
    else:
        print()
    n = len(out.token_ids)
    print(f"prompt {len(prompt_ids)} tokens; predict {n} tokens in {dt:.2f} s, {n / dt if dt > 0 else 0:.1f} t/s; "
          f"finish: {out.finish_reason}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
