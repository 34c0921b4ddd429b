"""``python -m atom_amd.examples.simple_inference --model DIR --temperature T --max-tokens N``
in the manner of atom/examples/simple_inference.py:15-95: every engine flag plus
``--temperature`` (0.6) and ``--max-tokens`` (300); prints each prompt and completion.
With a tokenizer that has a chat template every prompt is rendered as one user message with
the generation prompt appended (atom/examples/simple_inference.py:66-70).  Without a tokenizer in the model folder (random-weight folders have none) the prompts are
seeded random token ids and completions are printed as ids."""

from __future__ import annotations

import argparse
import random

from atom_amd import SamplingParams
from atom_amd.engine.arg_utils import EngineArgs, FlexibleArgumentParser

parser = FlexibleArgumentParser(formatter_class=argparse.RawTextHelpFormatter, description="simple offline inference")
EngineArgs.add_cli_args(parser)
parser.add_argument("--temperature", type=float, default=0.6, help="temperature for sampling")
parser.add_argument("--max-tokens", type=int, default=300, help="max sampled tokens per prompt")
parser.add_argument("--prompt-lens", type=str, default="5,17,33", help="lengths of the random-id prompts")


def render_chat(tokenizer, content: str) -> str:
    """The prompt as the model's chat template renders one user message, generation prompt included
    (atom/entrypoints/openai/chat_encoders.py:118-122); the text itself where the tokenizer has no template."""
    if not getattr(tokenizer, "chat_template", None):
        return content
    return tokenizer.apply_chat_template([{"role": "user", "content": content}], tokenize=False,
                                         add_generation_prompt=True)


def main(argv=None):
    args = parser.parse_args(argv)
    llm = EngineArgs.from_cli_args(args).create_engine()
    sampling_params = SamplingParams(temperature=args.temperature, max_tokens=args.max_tokens)
    if llm.tokenizer is not None:
        prompts = [render_chat(llm.tokenizer, p)
                   for p in ("introduce yourself", "list all prime numbers within 100", "1+2+3=?")]
    else:
        rng = random.Random(args.seed)
        vocab = llm.config.model_config.vocab_size
        prompts = [[rng.randrange(vocab) for _ in range(int(n))] for n in args.prompt_lens.split(",")]
    outputs = llm.generate(prompts, sampling_params)
    for prompt, output in zip(prompts, outputs):
        print("\n")
        print(f"Prompt: {prompt!r}")
        print(f"Completion: {(output['text'] or output['token_ids'])!r}")
        print(f"finish_reason={output['finish_reason']} ttft={output['ttft']:.4f}s tpot={output['tpot']:.4f}s")


if __name__ == "__main__":
    main()
