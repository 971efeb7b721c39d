"""Command line: generate from one prompt.

    python -m tokamak_amd.cli --model DIR --prompt-ids 1,2,3 --max-new-tokens 16
    python -m tokamak_amd.cli --random-weights tiny-a --prompt-ids 5,6,7 --temperature 0

Options ``--model --prompt --max-new-tokens --temperature --top-p`` and their
defaults are those of the reference's example (examples/basic_generation.py:14-20);
``--prompt`` needs a tokenizer in the folder and goes through the folder's chat template
(or the architecture's, if the folder has none); ``--prompt-ids`` needs neither.
"""

from __future__ import annotations

import argparse
import sys
import tempfile


def main(argv: list[str] | None = None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", default=None, help="model folder (config.json + safetensors)")
    parser.add_argument("--prompt", default="What does an LLM inference engine do?")
    parser.add_argument("--prompt-ids", default=None, help="comma-separated token ids (no tokenizer needed)")
    parser.add_argument("--max-new-tokens", type=int, default=256)
    parser.add_argument("--temperature", type=float, default=0.7)
    parser.add_argument("--top-p", type=float, default=0.95)
    parser.add_argument("--top-k", type=int, default=0)
    parser.add_argument("--seed", type=int, default=None)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--max-seq-len", type=int, default=None)
    parser.add_argument("--random-weights", default=None, metavar="PRESET",
                        help="write a folder of seeded random weights of this shape and use it")
    parser.add_argument("--weights-seed", type=int, default=0)
    parser.add_argument("--quiet", action="store_true", help="no load report and no progress bar")
    args = parser.parse_args(argv)

    from tokamak_amd import LLM, SamplingParams

    if not args.quiet:
        import logging

        logging.basicConfig(level=logging.INFO, format="%(name)s: %(message)s")
    if (args.model is None) == (args.random_weights is None):
        parser.error("give exactly one of --model and --random-weights")
    tmp = None
    folder = args.model
    if args.random_weights is not None:
        from tokamak_amd.config import find_preset, preset_names
        from tokamak_amd.weights import write_random_model

        if args.random_weights not in preset_names():
            parser.error(f"unknown preset {args.random_weights!r}; presets: {preset_names()}")
        _, config = find_preset(args.random_weights)
        tmp = tempfile.TemporaryDirectory(prefix="tokamak_amd_")
        folder = write_random_model(tmp.name, config, args.weights_seed)

    llm = LLM(folder, dtype=args.dtype, block_size=args.page_size, max_seq_len=args.max_seq_len)
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
                            max_new_tokens=args.max_new_tokens, seed=args.seed)
    if args.prompt_ids is not None:
        ids = [int(t) for t in args.prompt_ids.split(",") if t.strip()]
        outputs = llm.generate(prompt_token_ids=[ids], sampling_params=params, use_tqdm=not args.quiet)
        print(f"\n[prompt ids]\n{ids}\n")
    else:
        if llm.tokenizer is None:
            parser.error("the model folder has no tokenizer.json: use --prompt-ids")
        outputs = llm.generate(llm.chat_prompt(args.prompt), params, use_tqdm=not args.quiet)
        print(f"\n[prompt]\n{args.prompt}\n")
    out = outputs[0]
    print(f"[completion ({out.finish_reason.value})]")
    print(out.output_text if out.output_text is not None else out.output_token_ids)
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())
