"""Throughput of GPT-2 XL-sized generation on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers 48] [--dtype bf16]

With no flags, 16 untimed and 495 timed steps take the sequences from 512 to 1,024 tokens.

A step is one decode step of the whole batch: the engine's step function followed by greedy
selection and the readback of the chosen ids, exactly what the generation loop runs.  The
default run has the layer sizes of GPT-2 XL with random weights, a batch of 8 sequences that
were prefilled with 512 synthetic tokens each and are decoded to 1,024.  One JSON line
is printed:
  value      decoded tokens per second over the K timed steps
  prefill    one step of 2 x 1,024 prompt tokens: tokens/s, ms, fraction of the MFMA peak
  roofline   bytes a decode step has to read (every weight once + the live cache) / its time,
             against 8 TB/s
  points     decoded tokens per second at batch 1 and 64
"""

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

XL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 48, "n_embd": 1600, "n_head": 25,
      "n_inner": 6400, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
      "layer_norm_epsilon": 1e-5}
PROMPT_LEN, CONTEXT_LEN, PREFILL_SEQS, PREFILL_LEN = 512, 1024, 2, 1024


def build_model(config, dtype):
    """Random weights of the architecture, drawn on the GPU (std 0.02; norm scales around 1)."""
    import torch

    import burn_transformers_amd as bt
    family = bt.resolve_family(config)
    typed = family.config_class.from_dict(config)
    gen = torch.Generator(device="cuda:0").manual_seed(0)
    tensors = {}
    for spec in family.contract(typed).tensors:
        t = torch.randn(spec.shape, generator=gen, device="cuda:0", dtype=torch.float32) * 0.02
        if spec.layout == "vector" and spec.name.endswith("weight"):
            t += 1.0
        tensors[spec.name] = t.to(torch.bfloat16)
    return bt.model_from_tensors(config, tensors, dtype="bfloat16" if dtype == "bf16" else "float32")


def synthetic_prompts(batch, length, vocab, seed):
    import torch
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (batch, length), generator=gen).tolist()


def decode_run(engine, batch, warmup, steps, vocab):
    """(seconds for `steps` decode steps, mean context length over them)."""
    import torch

    import burn_transformers_amd as bt
    from burn_transformers_amd.sampling.sampler import Sampler
    steps = min(steps, CONTEXT_LEN - PROMPT_LEN - warmup - 1)
    prompts = synthetic_prompts(batch, PROMPT_LEN, vocab, seed=batch)
    slots = [engine.open() for _ in prompts]
    sampler = Sampler(bt.GenerationConfig(), batch, engine.device)
    rows = list(range(batch))
    # prefill in groups of at most 8 prompts to bound the workspace
    logits = torch.empty((batch, vocab), dtype=torch.float32, device=engine.device)
    for begin in range(0, batch, 8):
        part = engine.step([(slots[i], prompts[i]) for i in range(begin, min(begin + 8, batch))])
        logits[begin:begin + part.shape[0]] = part
    ids, _ = sampler.select(logits, rows)

    def one_step(ids):
        logits = engine.step([(slot, [token]) for slot, token in zip(slots, ids)])
        return sampler.select(logits, rows)[0]

    for _ in range(warmup):
        ids = one_step(ids)
    first_context = engine.length(slots[0])
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(steps):
        ids = one_step(ids)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    mean_context = first_context + (steps + 1) / 2.0     # keys each step's query reads, itself included
    for slot in slots:
        engine.close(slot)
    return elapsed, steps, mean_context


def prefill_run(engine, vocab, repeats=5):
    """Median seconds of one step of PREFILL_SEQS x PREFILL_LEN prompt tokens."""
    import torch
    prompts = synthetic_prompts(PREFILL_SEQS, PREFILL_LEN, vocab, seed=99)
    times = []
    for _ in range(repeats + 1):
        slots = [engine.open() for _ in prompts]
        torch.cuda.synchronize()
        started = time.perf_counter()
        engine.step(list(zip(slots, prompts)))
        torch.cuda.synchronize()
        times.append(time.perf_counter() - started)
        for slot in slots:
            engine.close(slot)
    times = sorted(times[1:])
    return times[len(times) // 2]


def model_bytes_and_flops(config, layers):
    d, m, v = config["n_embd"], config["n_inner"], config["vocab_size"]
    per_layer = 3 * d * d + d * d + 2 * d * m           # matrix elements
    vectors = 3 * d + d + m + d + 4 * d
    weight_bytes = 2 * (layers * per_layer + v * d) + 4 * (layers * vectors + 2 * d)
    kv_bytes_per_token = 2 * layers * d * 2
    dense = 2.0 * PREFILL_SEQS * PREFILL_LEN * layers * per_layer
    attention = layers * PREFILL_SEQS * 2.0 * d * PREFILL_LEN * (PREFILL_LEN + 1)
    readout = 2.0 * PREFILL_SEQS * d * v
    return weight_bytes, kv_bytes_per_token, dense + attention + readout


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=CONTEXT_LEN - PROMPT_LEN - 16 - 1)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=XL["n_layer"], help="fewer layers than the 48 of GPT-2 XL")
    parser.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    parser.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this library")
        sys.exit(2)
    import torch

    import burn_transformers_amd as bt

    config = dict(XL, n_layer=args.layers)
    model = build_model(config, args.dtype)
    vocab = config["vocab_size"]
    weight_bytes, kv_per_token, prefill_flops = model_bytes_and_flops(config, args.layers)
    engine = bt.Engine(model, max_tokens=max(args.batch, 64) * CONTEXT_LEN)

    elapsed, steps, mean_context = decode_run(engine, args.batch, args.warmup, args.steps, vocab)
    ms_per_step = 1000.0 * elapsed / steps
    value = args.batch * steps / elapsed
    step_bytes = weight_bytes + args.batch * mean_context * kv_per_token
    achieved = step_bytes / (elapsed / steps) / 1e9

    prefill_seconds = prefill_run(engine, vocab)
    prefill = {"value": round(PREFILL_SEQS * PREFILL_LEN / prefill_seconds, 1), "tokens": PREFILL_SEQS * PREFILL_LEN,
               "ms": round(1000.0 * prefill_seconds, 3),
               "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[args.dtype], 4)}
    points = {}
    if not args.no_points:
        for batch in (1, 64):
            e, s, _ = decode_run(engine, batch, args.warmup, args.steps, vocab)
            points[f"decode_b{batch}"] = round(batch * s / e, 1)

    print(json.dumps({
        "metric": f"decode tok/s at batch {args.batch} (GPT-2 XL sizes, 512-token prompts decoded to 1,024)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic token ids, random weights",
        "config": {"model": "gpt2-xl", "n_layer": args.layers, "n_layer_full": XL["n_layer"],
                   "n_embd": config["n_embd"], "n_head": config["n_head"], "n_inner": config["n_inner"],
                   "vocab_size": vocab, "n_positions": config["n_positions"], "global_batch": args.batch,
                   "prompt_len": PROMPT_LEN, "seq_len": CONTEXT_LEN, "mean_context": round(mean_context, 1),
                   "parallelism": "single GPU", "decode_graphs": True},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }))


if __name__ == "__main__":
    main()
