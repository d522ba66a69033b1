"""Command line in the manner of the reference's ``llama_generate`` example
(examples/llama_generate.rs:11, 66-81):

    gpt2_generate MODEL_DIR ["PROMPT"] [MAX_NEW_TOKENS]

MODEL_DIR holds config.json and safetensors weights; the class of model is the one config.json
names.  PROMPT defaults to "The three primary colors are" and MAX_NEW_TOKENS to 32; zero new
tokens or a fourth positional argument is a usage error, as there.  A prompt of text needs
``tokenizer.json`` in MODEL_DIR (the reference fails the same way without it); a prompt of
token ids (``464,1115,4165``; several prompts separated by ``;``) needs none.  Options carry
the names of the reference's GenerationConfig fields (src/generation.rs:191-276).
"""

import argparse
import json
import os
import re
import sys

USAGE = "usage: gpt2_generate MODEL_DIR [PROMPT] [MAX_NEW_TOKENS]"
DEFAULT_PROMPT = "The three primary colors are"


def parse_prompts(text, model_dir):
    """([token ids per prompt], tokenizer or None)."""
    if re.fullmatch(r"[\d\s,;]+", text):
        prompts = [[int(t) for t in part.replace(",", " ").split()] for part in text.split(";")]
        return [p for p in prompts if p], None
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        raise SystemExit("error: the model directory has no tokenizer.json; give the prompt as token ids (1,2,3)")
    from tokenizers import Tokenizer
    tokenizer = Tokenizer.from_file(path)
    return [tokenizer.encode(part).ids for part in text.split(";") if part], tokenizer


def main(argv=None):
    parser = argparse.ArgumentParser(prog="gpt2_generate", usage=USAGE + " [options]", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("model_dir")
    parser.add_argument("prompt", nargs="?", default=DEFAULT_PROMPT)
    parser.add_argument("max_new_tokens", nargs="?", type=int, default=32)
    parser.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    parser.add_argument("--strategy", choices=["greedy", "sample"], default=None,
                        help="default: greedy, or sample when --temperature, --top-k, --top-p or --min-p is given")
    parser.add_argument("--temperature", type=float, default=None)
    parser.add_argument("--seed", type=int, default=0, help="seed of the sampling stream")
    parser.add_argument("--min-new-tokens", type=int, default=0)
    parser.add_argument("--eos-token-ids", type=lambda s: [int(t) for t in s.split(",") if t], default=[])
    parser.add_argument("--stop-sequences", type=lambda s: [[int(t) for t in q.split(",") if t] for q in s.split(";")],
                        default=[], help="token-id sequences, e.g. 13,198;50256")
    parser.add_argument("--top-k", type=int, default=None, help="sampling: keep scores >= the k-th greatest")
    parser.add_argument("--top-p", type=float, default=None, help="sampling: nucleus mass in (0, 1]")
    parser.add_argument("--min-p", type=float, default=None, help="sampling: keep p >= min_p * max p")
    parser.add_argument("--repetition-penalty", type=float, default=1.0)
    parser.add_argument("--presence-penalty", type=float, default=0.0)
    parser.add_argument("--frequency-penalty", type=float, default=0.0)
    parser.add_argument("--additive-penalty-scope", choices=["generated", "prompt_and_generated"], default="generated")
    parser.add_argument("--no-repeat-ngram-size", type=int, default=0)
    parser.add_argument("--logit-bias", default={}, help="token:bias pairs, e.g. 50256:-100,13:1.5",
                        type=lambda s: {int(k): float(v) for k, v in (pair.split(":") for pair in s.split(",") if pair)})
    parser.add_argument("--total-length", type=int, default=None,
                        help="a sequence also ends when prompt and output together hold this many tokens")
    parser.add_argument("--prefill-chunk-size", type=int, default=None)
    parser.add_argument("--batch-size", type=int, default=None, help="most prompts that start together")
    parser.add_argument("--max-tokens", type=int, default=None, help="cache size in tokens (default: what the prompts need)")
    parser.add_argument("--random-weights", metavar="CONFIG.json", default=None,
                        help="first write MODEL_DIR from this configuration with random weights")
    parser.add_argument("--weights-seed", type=int, default=0)
    parser.add_argument("--json", action="store_true", help="print one JSON object per sequence")
    parser.add_argument("--load-report", action="store_true",
                        help="print to stderr what loading did with the checkpoint's tensors (one JSON object)")
    args, extra = parser.parse_known_args(argv)
    if extra or args.max_new_tokens == 0:
        print(USAGE, file=sys.stderr)
        return 2

    import burn_transformers_amd as bt
    if args.random_weights:
        with open(args.random_weights) as handle:
            bt.write_random_model(args.model_dir, json.load(handle), args.weights_seed)
    prompts, tokenizer = parse_prompts(args.prompt, args.model_dir)
    wants_sampling = any(v is not None for v in (args.temperature, args.top_k, args.top_p, args.min_p))
    strategy = args.strategy or ("sample" if wants_sampling else "greedy")
    config = bt.GenerationConfig(
        max_new_tokens=args.max_new_tokens, min_new_tokens=args.min_new_tokens, strategy=strategy,
        temperature=args.temperature if args.temperature is not None else 1.0, seed=args.seed,
        eos_token_ids=args.eos_token_ids, stop_sequences=args.stop_sequences, top_k=args.top_k, top_p=args.top_p,
        min_p=args.min_p, repetition_penalty=args.repetition_penalty, presence_penalty=args.presence_penalty,
        frequency_penalty=args.frequency_penalty, additive_penalty_scope=args.additive_penalty_scope,
        no_repeat_ngram_size=args.no_repeat_ngram_size, logit_bias=args.logit_bias)
    model = bt.load_model(args.model_dir, dtype=args.dtype)
    if args.load_report:
        print(json.dumps(model.load_report), file=sys.stderr)
    grows_to = lambda n: n + args.max_new_tokens if args.total_length is None else min(n + args.max_new_tokens, args.total_length)
    need = sum((grows_to(len(p)) + 63) // 64 * 64 for p in prompts)
    engine = bt.Engine(model, max_tokens=args.max_tokens or need)
    sequences = bt.generate(engine, prompts, config, prefill_chunk=args.prefill_chunk_size,
                            batch_size=args.batch_size, total_length=args.total_length)
    for prompt, sequence in zip(prompts, sequences):
        if args.json:
            print(json.dumps({"prompt_length": sequence.prompt_length, "token_ids": sequence.token_ids,
                              "log_probabilities": sequence.log_probabilities,
                              "finish_reason": str(sequence.finish_reason)}))
        elif tokenizer is not None:
            print(tokenizer.decode(prompt + sequence.token_ids))
        else:
            print(",".join(str(t) for t in sequence.token_ids) + f"    [{sequence.finish_reason}]")
    return 0


if __name__ == "__main__":
    sys.exit(main())
