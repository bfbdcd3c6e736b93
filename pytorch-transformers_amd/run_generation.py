"""Text generation from the command line, with the option names of the reference's example.

    python -m pytorch_transformers_amd.run_generation --model_name_or_path DIR --prompt_ids 3,1,4 --length 20

Options shared with examples/pytorch/text-generation/run_generation.py:286-333 keep its names,
defaults and meanings: ``--model_type``, ``--model_name_or_path``, ``--prompt``, ``--length`` (20),
``--stop_token``, ``--temperature`` (1.0), ``--repetition_penalty`` (1.0), ``--k`` (0), ``--p``
(0.9), ``--prefix``, ``--seed`` (42), ``--num_return_sequences`` (1).  Like it, the program samples
(``do_sample=True``, :408-417) and prints ``=== GENERATED SEQUENCE n ===`` before each result
(:425-441).  Added here: ``--prompt_ids`` / ``--prompt_file`` (token ids, for folders without a
tokenizer), ``--greedy``, ``--dtype``, ``--random_config`` with ``--random_seed`` (write a model
folder with random weights first), ``--min_length``-style limits and ``--batch_size``; ``--tune`` (time, once,
the choices between kernels that no rule decides, for this run's prompt lengths and batch, before anything is
generated) and ``--tuning_table FILE`` (such choices as a JSON file: read if it is there, written after ``--tune``),
with which a run makes the choices of the run that was measured.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile

def new_token_budget(length: int, context: int, longest_prompt: int) -> int:
    """New tokens for ``--length``.  The reference's example caps the request at the model's trained context and
    reads a negative length as "as long as the model allows" (run_generation.py:151-158, :371-376).  Here the
    sequence as a whole stays within the trained context where the configuration names one; nothing else limits
    it, because the cache is sized for what is asked."""
    room = max(1, context - longest_prompt) if context > 0 else None
    if length < 0:
        if room is None:
            raise ValueError("--length is negative and the configuration names no context length to fill")
        return room
    return length if room is None else min(length, room)


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(description="Generate text (or token ids) with a model folder on one AMD GPU")
    ap.add_argument("--model_type", default=None, type=str, help="checked against config.json's model_type if given")
    ap.add_argument("--model_name_or_path", default=None, type=str, help="folder with config.json and model.safetensors")
    ap.add_argument("--prompt", type=str, default="")
    ap.add_argument("--prompt_ids", type=str, default=None, help="comma-separated token ids; ';' separates prompts")
    ap.add_argument("--prompt_file", type=str, default=None, help="file with one prompt of comma-separated ids per line")
    ap.add_argument("--length", type=int, default=20)
    ap.add_argument("--min_new_tokens", type=int, default=None)
    ap.add_argument("--stop_token", type=str, default=None, help="text at which the printed result is cut")
    ap.add_argument("--stop_token_id", type=int, action="append", default=None, help="token id that ends a sequence")
    ap.add_argument("--temperature", type=float, default=1.0,
                    help="temperature of 1.0 has no effect, lower tend toward greedy sampling")
    ap.add_argument("--repetition_penalty", type=float, default=1.0)
    ap.add_argument("--k", type=int, default=0)
    ap.add_argument("--p", type=float, default=0.9)
    ap.add_argument("--min_p", type=float, default=None)
    ap.add_argument("--greedy", action="store_true", help="argmax instead of sampling")
    ap.add_argument("--prefix", type=str, default="", help="Text added prior to input.")
    ap.add_argument("--seed", type=int, default=42, help="random seed for sampling")
    ap.add_argument("--num_return_sequences", type=int, default=1, help="The number of samples to generate.")
    ap.add_argument("--batch_size", type=int, default=None, help="prompts per batch; further batches follow")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--fp16", action="store_true", help="accepted for compatibility; the 16-bit type here is bfloat16")
    ap.add_argument("--device", default="cuda:0")
    # options of the reference's example that have no counterpart here: accepted where they change nothing, refused where
    # they would (examples/pytorch/text-generation/run_generation.py:316-332)
    ap.add_argument("--padding_text", type=str, default="", help="Deprecated, the use of `--prefix` is preferred.")
    ap.add_argument("--xlm_language", type=str, default="",
                    help="the reference's language choice for XLM; must stay empty: Falcon has none")
    ap.add_argument("--use_cpu", action="store_true", help="refused: the model runs on the GPU only")
    ap.add_argument("--jit", action="store_true",
                    help="accepted for compatibility: nothing is traced; decode steps are captured as HIP graphs anyway")
    ap.add_argument("--random_config", type=str, default=None, help="config.json to build a random-weights model from")
    ap.add_argument("--random_seed", type=int, default=0)
    ap.add_argument("--tune", action="store_true",
                    help="time the choices between kernels for this run's prompt lengths and batch before generating")
    ap.add_argument("--tuning_table", type=str, default=None,
                    help="JSON file of timed choices: taken if it exists; written after --tune")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.use_cpu:
        print("--use_cpu: there is no CPU path; the model runs on an AMD GPU (see --device)", file=sys.stderr)
        return 2
    if args.xlm_language:
        print("--xlm_language belongs to another architecture of the reference's example and would change nothing here; "
              "leave it out", file=sys.stderr)
        return 2
    if not args.prefix:  # the older name of the same option (run_generation.py:382)
        args.prefix = args.padding_text
    from . import AutoConfig, GenerationConfig
    from .pipeline import pipeline
    from .weights import write_random_model

    tmp = None
    folder = args.model_name_or_path
    if args.random_config is not None:
        tmp = tempfile.TemporaryDirectory()
        with open(args.random_config) as f:
            cfg = AutoConfig.from_dict(json.load(f))
        folder = write_random_model(tmp.name, cfg, args.random_seed)
    if folder is None:
        print("one of --model_name_or_path and --random_config is required", file=sys.stderr)
        return 2
    config = AutoConfig.from_pretrained(folder)
    if args.model_type is not None and args.model_type != config.model_type:
        print(f"--model_type {args.model_type} but {folder} holds model_type {config.model_type}", file=sys.stderr)
        return 2
    table = args.tuning_table if args.tuning_table and os.path.isfile(args.tuning_table) else None
    pipe = pipeline("text-generation", model=folder, dtype=args.dtype, device=args.device, tuning_table=table)

    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts = [[int(t) for t in line.replace(",", " ").split()] for line in f if line.strip()]
    elif args.prompt_ids:
        prompts = [[int(t) for t in part.replace(",", " ").split()] for part in args.prompt_ids.split(";")]
    else:
        text = args.prompt if args.prompt else input("Model prompt >>> ")  # run_generation.py:365
        prompts = [text]

    longest = max((len(p) for p in prompts if not isinstance(p, str)), default=0)
    length = new_token_budget(args.length, int(getattr(config, "max_position_embeddings", 0) or 0), longest)
    gen = dict(max_new_tokens=length, min_new_tokens=args.min_new_tokens, seed=args.seed,
               repetition_penalty=args.repetition_penalty, num_return_sequences=args.num_return_sequences)
    if args.stop_token_id is not None:
        gen["eos_token_id"] = args.stop_token_id
    if args.greedy:
        gen.update(do_sample=False, num_return_sequences=1)
    else:
        gen.update(do_sample=True, temperature=args.temperature, top_k=args.k, top_p=args.p, min_p=args.min_p)
    GenerationConfig(**{k: v for k, v in gen.items()})  # validate before the model runs
    if args.tune:
        lens = [len(pipe._encode(p, args.prefix)) for p in prompts]
        rows = len(prompts) * (gen["num_return_sequences"] or 1)
        batch = min(rows, args.batch_size) if args.batch_size else rows
        mean = sum(lens) // len(lens)
        timed = pipe.model.tune(prompt_lens=sorted(set(lens)), batches=(batch,),
                                contexts=((max(lens) + 1, mean + 1), (max(lens) + length, mean + length)))
        if args.tuning_table:
            with open(args.tuning_table, "w") as f:
                json.dump(timed, f)
    results = pipe(prompts, prefix=args.prefix, batch_size=args.batch_size, **gen)
    n = 0
    for records in results:
        for rec in records:
            n += 1
            print(f"=== GENERATED SEQUENCE {n} ===")
            if "generated_text" in rec:
                text = rec["generated_text"]
                if args.stop_token:
                    text = text[: text.find(args.stop_token) if args.stop_token in text else None]  # :433
                print(text)
            else:
                print(",".join(str(t) for t in rec["generated_token_ids"]))
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
