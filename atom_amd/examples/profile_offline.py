"""``python -m atom_amd.examples.profile_offline --model DIR --input-length N --output-length M --bs B``
in the manner of atom/examples/profile_offline.py:12-117: every engine flag plus ``--input-length`` (128),
``--output-length`` (32), ``--bs`` (1) and ``--random-input``.  One short request warms the engine up, then
``--bs`` equal prompts are generated between ``start_profile`` and ``stop_profile`` and the trace is written to
``--torch-profiler-dir`` (``./profiler_traces`` when it is not given, as there).  With ``--random-input``, or
when the model folder has no tokenizer (random-weight folders have none), the prompt is ``--input-length`` seeded
random token ids; otherwise a fixed text."""

from __future__ import annotations

import argparse
import random

from atom_amd import SamplingParams
from atom_amd.engine.arg_utils import EngineArgs, FlexibleArgumentParser

DEFAULT_TRACE_DIR = "./profiler_traces"
FIXED_PROMPT = ("Paged caches keep the keys and values of every request in blocks of a fixed number of tokens. "
                "Describe how a scheduler that admits requests under a token budget decides which blocks to give "
                "back when the pool runs out, and what that costs the request that loses them.")

parser = FlexibleArgumentParser(formatter_class=argparse.RawTextHelpFormatter,
                                description="offline profiling of one batch of equal requests")
EngineArgs.add_cli_args(parser)
parser.add_argument("--input-length", type=int, default=128, help="prompt length in tokens (with --random-input)")
parser.add_argument("--output-length", type=int, default=32, help="tokens generated per request")
parser.add_argument("--bs", type=int, default=1, help="number of requests generated together")
parser.add_argument("--random-input", action="store_true", help="random token ids instead of the fixed text")


def make_prompt(llm, args):
    """The one prompt of the run: token ids when random, text otherwise."""
    if args.random_input or llm.tokenizer is None:
        rng = random.Random(args.seed)
        vocab = llm.config.model_config.vocab_size
        return [rng.randrange(vocab) for _ in range(args.input_length)]
    return FIXED_PROMPT


def main(argv=None):
    args = parser.parse_args(argv)
    if args.input_length < 1 or args.output_length < 1 or args.bs < 1:
        parser.error("--input-length, --output-length and --bs must be positive")
    if args.torch_profiler_dir is None:
        args.torch_profiler_dir = DEFAULT_TRACE_DIR
        print(f"Warning: --torch-profiler-dir not specified, using default: {DEFAULT_TRACE_DIR}")
    llm = EngineArgs.from_cli_args(args).create_engine()
    prompt = make_prompt(llm, args)
    sampling_params = SamplingParams(temperature=0.6, max_tokens=args.output_length, ignore_eos=True)
    print("Warming up...")
    llm.generate([prompt[:8] if isinstance(prompt, list) else "warmup"], sampling_params)
    print("Warm up done")
    llm.start_profile()
    print(f"Processing batch of {args.bs} requests...")
    outputs = llm.generate([prompt] * args.bs, sampling_params)
    llm.stop_profile()
    print("Profiler traces have been saved to:", args.torch_profiler_dir)
    for i, output in enumerate(outputs):
        print(f"Output [{i + 1}/{args.bs}]: {(output['text'] or output['token_ids'])!r}")
    return outputs


if __name__ == "__main__":
    main()
