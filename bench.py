"""Throughput of GPT-2 generation on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers 48] [--dtype bf16]
                    [--repetitions 10] [--workload xl|small|medium|sweep] [--model xl|medium|small]
                    [--kernel-batches 1,64] [--sweep-part all|decode|prompts] [--no-points] [--no-kernels] [--no-own]

The default workload (``xl``) has the layer sizes of GPT-2 XL with random weights: a batch of 8
sequences, prefilled with 512 synthetic tokens each, is decoded towards 1,024.  A step is one
decode step of the whole batch: the engine's step function, greedy selection and the readback of
the chosen ids, exactly what the generation loop runs (the ids feed the next step from the GPU,
and the host reads them while that step runs).  With no flags, 16 untimed and
495 timed steps take the sequences from 512 to 1,024 tokens.

The protocol is the reference's (BENCHMARKS.md:71-87, tests/support/causal_decode_benchmark.rs:
1-31): 3 warm-up repetitions and 10 measured ones, every repetition on fresh sequences (new slots,
a new prefill), the device synchronised at both ends of the timed steps, forced length (no end
token), real tokens only; the median repetition is the value, the fastest and slowest are given.

One JSON line is printed:
  value       decoded tokens per second over the K timed steps of the median repetition
  spread      milliseconds per step of the fastest, median and slowest repetition
  prefill     one step of 2 x 1,024 prompt tokens: tokens/s, ms, fraction of the MFMA peak;
              `own` is the same step with every product on this package's kernels (the default
              hands products of more than 256 rows, 512 for those that add to the residual
              stream, to hipBLASLt, as the reference hands its products to its backend's library)
  roofline    bytes a decode step has to read (every weight once + the live cache) / its time,
              against 8 TB/s
  points      decoded tokens per second at batch 1 and 64, at batch 8 from prompts of 896 tokens
              (contexts up to the position limit), and prompt tokens per second of 2 x 1,024
              prompt tokens fed in chunks of 256 (eight steps of 2 x 256 tokens)
  kernels     for the decode step and for the prefill step, each class of kernel on its own: the
              step's launch list is cut into classes (same kernel, same shape), each class's calls
              (one per layer, every layer's own weights) are replayed alone from a HIP graph and
              timed with events; per call: microseconds and the fraction of the HBM roofline
              (decode) or of the MFMA peak (prefill)

``--model medium`` / ``--model small`` run the same measurement (same JSON line) at the layer sizes
of GPT-2 medium and small; ``--kernel-batches 1,64`` adds the kernel classes of decode steps of
those batch sizes beside the main one (``kernels.decode_b1`` ...).

``--workload small`` and ``--workload medium`` run the other two measured workloads through the
generation loop: GPT-2 small sizes in float32, 16 prompts of 1 to 1,000 tokens decoded greedily to
1,024 tokens each; GPT-2 medium sizes, 64 prompts of 64 to 768 tokens prefilled in chunks of 256
and sampled at temperature 1 to 1,024 tokens each.  Their value is generated tokens per second.
``--workload sweep`` prints a table of further sizes (decode over batch sizes and contexts up to
8,192 tokens, prompts of 64 to 8,192 tokens whole and in chunks of 256) instead of the JSON line.
"""

import argparse
import json
import statistics
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
ELEMENT_BYTES = {"bf16": 2, "fp32": 4}

XL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 48, "n_embd": 1600, "n_head": 25,
      "n_inner": 6400, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
      "layer_norm_epsilon": 1e-5}
SMALL = dict(XL, n_layer=12, n_embd=768, n_head=12, n_inner=3072)
MEDIUM = dict(XL, n_layer=24, n_embd=1024, n_head=16, n_inner=4096)
MODELS = {"xl": XL, "medium": MEDIUM, "small": SMALL}
MODEL_NAMES = {"xl": "XL", "medium": "medium", "small": "small"}
PROMPT_LEN, CONTEXT_LEN, PREFILL_SEQS, PREFILL_LEN = 512, 1024, 2, 1024
WARMUP_REPETITIONS = 3


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


def decode_repetition(engine, batch, warmup, steps, vocab, seed, prompt_len=PROMPT_LEN):
    """One repetition on fresh sequences: (seconds of the timed steps, first context length)."""
    import torch

    import burn_transformers_amd as bt
    from burn_transformers_amd.engine.generate import select_and_step_ahead
    from burn_transformers_amd.sampling.sampler import Sampler
    prompts = synthetic_prompts(batch, prompt_len, vocab, seed=seed)
    slots = [engine.open() for _ in prompts]
    sampler = Sampler(bt.GenerationConfig(), batch, engine.device)
    rows = list(range(batch))
    # prefill in groups of at most 8 prompts to bound the workspace
    logits = torch.empty((batch, vocab), dtype=torch.float32, device=engine.device)
    for begin in range(0, batch, 8):
        part = engine.step([(slots[i], prompts[i]) for i in range(begin, min(begin + 8, batch))])
        logits[begin:begin + part.shape[0]] = part

    def run(count, logits):
        # the generation loop's own turn: the selection is started, its ids feed the next step from
        # the GPU, and the host reads them (the step's one readback) while that step runs
        for _ in range(count):
            _, _, logits = select_and_step_ahead(engine, sampler, slots, logits, rows, rows)
        return logits

    logits = run(warmup, logits)
    first_context = engine.length(slots[0])
    torch.cuda.synchronize()
    started = time.perf_counter()
    run(steps, logits)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    for slot in slots:
        engine.close(slot)
    return elapsed, first_context


def decode_run(engine, batch, warmup, steps, vocab, repetitions, warmup_repetitions=WARMUP_REPETITIONS,
               prompt_len=PROMPT_LEN):
    """(sorted seconds of the measured repetitions, steps, mean context length over the timed steps)."""
    steps = max(1, min(steps, CONTEXT_LEN - prompt_len - warmup - 1))
    for r in range(warmup_repetitions):          # short: they are there for graphs, clocks and caches
        decode_repetition(engine, batch, warmup, min(steps, 24), vocab, 1000 + r, prompt_len)
    times, first_context = [], prompt_len
    for r in range(repetitions):
        elapsed, first_context = decode_repetition(engine, batch, warmup, steps, vocab, batch * 100 + r, prompt_len)
        times.append(elapsed)
    mean_context = first_context + (steps + 1) / 2.0     # keys each step's query reads, itself included
    return sorted(times), steps, mean_context


def prefill_run(engine, vocab, repetitions, chunk=None):
    """Sorted seconds of PREFILL_SEQS x PREFILL_LEN prompt tokens on fresh sequences: in one step, or
    in steps of ``chunk`` tokens of every sequence."""
    import torch
    times = []
    for r in range(WARMUP_REPETITIONS + repetitions):
        prompts = synthetic_prompts(PREFILL_SEQS, PREFILL_LEN, vocab, seed=99 + r)
        slots = [engine.open() for _ in prompts]
        torch.cuda.synchronize()
        started = time.perf_counter()
        for begin in range(0, PREFILL_LEN, chunk or PREFILL_LEN):
            engine.step([(slot, prompt[begin:begin + (chunk or PREFILL_LEN)]) for slot, prompt in zip(slots, prompts)])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - started)
        for slot in slots:
            engine.close(slot)
    return sorted(times[WARMUP_REPETITIONS:])


def model_bytes_and_flops(config, layers, dtype):
    """(bytes of every weight a step reads, bytes of keys and values per cached token, flops of the
    prefill step): matrices and the cache in the element type of the run, vectors in float32."""
    d, m, v = config["n_embd"], config["n_inner"], config["vocab_size"]
    element = ELEMENT_BYTES[dtype]
    per_layer = 3 * d * d + d * d + 2 * d * m           # matrix elements
    vectors = 3 * d + d + m + d + 4 * d
    weight_bytes = element * (layers * per_layer + v * d) + 4 * (layers * vectors + 2 * d)
    kv_bytes_per_token = 2 * layers * d * element
    dense = 2.0 * PREFILL_SEQS * PREFILL_LEN * layers * per_layer
    attention = layers * PREFILL_SEQS * 2.0 * d * PREFILL_LEN * (PREFILL_LEN + 1)
    readout = 2.0 * PREFILL_SEQS * d * v
    return weight_bytes, kv_bytes_per_token, dense + attention + readout


# --- each class of kernel on its own -----------------------------------------------------------

def _class_of(name, call):
    """(label, bytes a call has to read, flops it does) of one recorded kernel call."""
    short = name[len("bt_"):-len("_call")]
    if short.startswith("gemm"):
        element = 4 if call.dtype == 0 else 2
        weights = call.N * call.K * element
        rows = call.M * call.K * (4 if call.has_norm else element)
        return f"{short} {call.M}x{call.N}x{call.K}", weights + rows, 2.0 * call.M * call.N * call.K
    if short.startswith("attention"):
        return f"{short} {call.args.n_tokens}tok", None, None       # filled in by the caller, who knows the contexts
    if short == "add_norm":
        return f"add_norm {call.n_rows}x{call.width}", (call.n_delta + 2) * call.n_rows * call.width * 4, 0.0
    if short == "embed":
        return f"embed {call.tokens}x{call.width}", call.tokens * call.width * 6, 0.0
    if short == "kv_copy":
        return f"kv_copy {call.tokens}tok", call.tokens * call.kv.kv_heads * call.kv.head_dim * 8, 0.0
    return short, 0, 0.0


def kernel_classes(engine, entries, attention_bytes, attention_flops, peak_flops, replays=20):
    """Runs one step of ``entries`` to get its launch list, then replays each class of calls alone
    from a HIP graph.  Returns {label: {"n": calls a step, "us": per call, "hbm": fraction of the
    HBM roofline, "mfma": fraction of the MFMA peak}}."""
    import torch
    from burn_transformers_amd.kernels import library as K
    if not engine.use_programs:
        return {}
    graphs, engine.use_graphs = engine.use_graphs, False
    before = [engine.length(slot) for slot, _ in entries]
    try:
        for attempt in range(3):     # a step that made a workspace grow leaves no list: it is rewound and run again
            engine.step(entries)
            torch.cuda.synchronize()
            if engine.last_program is not None:
                break
            for (slot, _), length in zip(entries, before):
                engine.truncate(slot, length)
    finally:
        engine.use_graphs = graphs
    program = engine.last_program
    if program is None:
        return {}
    classes = {}
    for lib, name, call in program.calls:
        label, nbytes, flops = _class_of(name, call)
        if nbytes is None:
            nbytes, flops = attention_bytes, attention_flops
        classes.setdefault(label, []).append((lib, name, call, nbytes, flops))
    out = {}
    for label, calls in classes.items():
        part = K.Program()
        repeat = -(-8 // len(calls))                 # a class of one or two calls is run eight times over:
        for _ in range(repeat):                      # a graph of a single kernel measures the graph's launch
            for lib, name, call, _, _ in calls:
                part.add(lib, name, call)
        part.run()                                   # once outside a graph (first-use set-up of a kernel)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            part.run()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        times = []
        for _ in range(replays):
            begin.record()
            graph.replay()
            end.record()
            end.synchronize()
            times.append(begin.elapsed_time(end) * 1e-3 / len(part))
        seconds = statistics.median(times)
        nbytes, flops = calls[0][3], calls[0][4]
        out[label] = {"n": len(calls), "us": round(seconds * 1e6, 2),
                      "hbm": round(nbytes / seconds / 1e9 / PEAK_HBM_GBS, 3),
                      "mfma": round(flops / seconds / peak_flops, 3)}
    return out


def decode_kernels(engine, batch, vocab, config, dtype, context):
    """Classes of a decode step of ``batch`` sequences that hold ``context`` tokens each."""
    prompts = synthetic_prompts(batch, context - 1, vocab, seed=7)
    slots = [engine.open() for _ in prompts]
    for begin in range(0, batch, 8):
        engine.step([(slots[i], prompts[i]) for i in range(begin, min(begin + 8, batch))])
    d = config["n_embd"]
    kv_bytes = batch * context * 2 * d * ELEMENT_BYTES[dtype]        # one layer's keys and values of the live context
    try:
        return kernel_classes(engine, [(slot, [5]) for slot in slots], kv_bytes, 4.0 * batch * context * d,
                              PEAK_FLOPS[dtype])
    finally:
        for slot in slots:
            engine.close(slot)


def prefill_kernels(engine, vocab, config, dtype):
    prompts = synthetic_prompts(PREFILL_SEQS, PREFILL_LEN, vocab, seed=8)
    slots = [engine.open() for _ in prompts]
    d = config["n_embd"]
    tokens = PREFILL_SEQS * PREFILL_LEN
    try:
        return kernel_classes(engine, list(zip(slots, prompts)), 4 * tokens * d * ELEMENT_BYTES[dtype],
                              PREFILL_SEQS * 2.0 * d * PREFILL_LEN * (PREFILL_LEN + 1), PEAK_FLOPS[dtype], replays=10)
    finally:
        for slot in slots:
            engine.close(slot)


# --- the workloads -----------------------------------------------------------------------------

def run_xl(args):
    import torch  # noqa: F401

    import burn_transformers_amd as bt
    from burn_transformers_amd.kernels import library as K

    config = dict(MODELS[args.model], n_layer=args.layers)
    model = build_model(config, args.dtype)
    vocab = config["vocab_size"]
    weight_bytes, kv_per_token, prefill_flops = model_bytes_and_flops(config, args.layers, args.dtype)
    engine = bt.Engine(model, max_tokens=max(args.batch, 64) * CONTEXT_LEN)

    times, steps, mean_context = decode_run(engine, args.batch, args.warmup, args.steps, vocab, args.repetitions)
    median = statistics.median(times)
    ms_per_step = 1000.0 * median / steps
    value = args.batch * steps / median
    step_bytes = weight_bytes + args.batch * mean_context * kv_per_token
    achieved = step_bytes / (median / steps) / 1e9
    final_context = PROMPT_LEN + args.warmup + steps + 1
    from_graphs = engine.graph_replays > 0       # the engine's own choice: a graph only where launching is the limit

    prefill_times = prefill_run(engine, vocab, args.repetitions)
    prefill_seconds = statistics.median(prefill_times)
    prefill = {"value": round(PREFILL_SEQS * PREFILL_LEN / prefill_seconds, 1), "tokens": PREFILL_SEQS * PREFILL_LEN,
               "ms": round(1000.0 * prefill_seconds, 3),
               "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[args.dtype], 4),
               "min_ms": round(1000.0 * prefill_times[0], 3), "max_ms": round(1000.0 * prefill_times[-1], 3),
               "products": "hipBLASLt beyond 256 rows" if args.dtype == "bf16" and K.library_products() else "own kernels"}
    kernels = {}
    if not args.no_kernels:
        kernels["decode"] = decode_kernels(engine, args.batch, vocab, config, args.dtype, int(mean_context))
        for batch in args.kernel_batches:
            kernels[f"decode_b{batch}"] = decode_kernels(engine, batch, vocab, config, args.dtype, int(mean_context))
        kernels["prefill"] = prefill_kernels(engine, vocab, config, args.dtype)
    if args.dtype == "bf16" and K.library_products() is not None and not args.no_own:
        # the same step with every product on this package's own kernels
        held = dict(K._library_state)
        K._library_state.update(tried=True, lib=None)
        try:
            own_engine = bt.Engine(model, max_tokens=PREFILL_SEQS * PREFILL_LEN)
            own = statistics.median(prefill_run(own_engine, vocab, max(3, args.repetitions // 2)))
            prefill["own"] = {"value": round(PREFILL_SEQS * PREFILL_LEN / own, 1), "ms": round(1000.0 * own, 3),
                              "frac": round(prefill_flops / own / PEAK_FLOPS[args.dtype], 4)}
            del own_engine
        finally:
            K._library_state.update(held)

    points = {}
    if not args.no_points:
        for batch in (1, 64):
            t, s, _ = decode_run(engine, batch, args.warmup, args.steps, vocab, max(3, args.repetitions // 2), 1)
            points[f"decode_b{batch}"] = round(batch * s / statistics.median(t), 1)
        # contexts near the position limit: batch 8 from prompts of 896 tokens towards 1,024
        t, s, _ = decode_run(engine, 8, args.warmup, args.steps, vocab, max(3, args.repetitions // 2), 1, prompt_len=896)
        points["decode_b8_from896"] = round(8 * s / statistics.median(t), 1)
        # the same 2 x 1,024 prompt tokens as `prefill`, fed in chunks of 256 tokens of each sequence
        chunked = statistics.median(prefill_run(engine, vocab, max(3, args.repetitions // 2), chunk=256))
        points["prefill_2x1024_chunks256"] = round(PREFILL_SEQS * PREFILL_LEN / chunked, 1)

    return {
        "metric": f"decode tok/s at batch {args.batch} (GPT-2 {MODEL_NAMES[args.model]} sizes, 512-token prompts decoded to "
                  f"{final_context} tokens, median of {args.repetitions} repetitions)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic token ids, random weights",
        "config": {"model": "gpt2-" + args.model, "n_layer": args.layers, "n_layer_full": MODELS[args.model]["n_layer"],
                   "n_embd": config["n_embd"], "n_head": config["n_head"], "n_inner": config["n_inner"],
                   "vocab_size": vocab, "n_positions": config["n_positions"], "global_batch": args.batch,
                   "prompt_len": PROMPT_LEN, "seq_len": CONTEXT_LEN, "final_context": final_context,
                   "mean_context": round(mean_context, 1), "parallelism": "single GPU", "decode_graphs": from_graphs,
                   "repetitions": args.repetitions, "warmup_repetitions": WARMUP_REPETITIONS},
        "spread": {"min_ms": round(1000.0 * times[0] / steps, 4), "median_ms": round(ms_per_step, 4),
                   "max_ms": round(1000.0 * times[-1] / steps, 4)},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
        "kernels": kernels,
    }


def run_generation(args):
    """The small and the medium workload through the generation loop."""
    import torch

    import burn_transformers_amd as bt
    if args.workload == "small":
        config, count, low, high, chunk, dtype = SMALL, 16, 1, 1000, None, args.dtype or "fp32"
        generation = bt.GenerationConfig(max_new_tokens=CONTEXT_LEN)
        what = "GPT-2 small sizes, 16 prompts of 1 to 1,000 tokens decoded greedily to 1,024 tokens each"
    else:
        config, count, low, high, chunk, dtype = MEDIUM, 64, 64, 768, 256, args.dtype or "bf16"
        generation = bt.GenerationConfig(max_new_tokens=CONTEXT_LEN, strategy="sample", temperature=1.0, seed=1)
        what = ("GPT-2 medium sizes, 64 prompts of 64 to 768 tokens prefilled in chunks of 256 and sampled at "
                "temperature 1 to 1,024 tokens each")
    model = build_model(config, dtype)
    engine = bt.Engine(model, max_tokens=count * CONTEXT_LEN)
    gen = torch.Generator().manual_seed(17)
    times, generated, prompt_tokens = [], 0, 0
    repetitions = max(3, args.repetitions // 2)
    for r in range(1 + repetitions):
        lengths = torch.randint(low, high + 1, (count,), generator=gen).tolist()
        prompts = [torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist() for n in lengths]
        torch.cuda.synchronize()
        started = time.perf_counter()
        out = bt.generate(engine, prompts, generation, prefill_chunk=chunk, total_length=CONTEXT_LEN)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        if r:                                        # the first repetition warms up
            times.append((elapsed, sum(len(s.token_ids) for s in out), sum(lengths)))
    times.sort(key=lambda t: t[1] / t[0])
    elapsed, generated, prompt_tokens = times[len(times) // 2]
    return {
        "metric": f"generated tok/s ({what}; median of {repetitions} repetitions)",
        "value": round(generated / elapsed, 1), "unit": "tokens/s", "n_gpus": 1, "steps": generated // count,
        "warmup": 1, "ms_per_step": round(1000.0 * elapsed / max(1, CONTEXT_LEN - low), 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic token ids, random weights",
        "config": {"model": "gpt2-" + args.workload, "n_layer": config["n_layer"], "n_embd": config["n_embd"],
                   "n_head": config["n_head"], "n_inner": config["n_inner"], "vocab_size": config["vocab_size"],
                   "n_positions": config["n_positions"], "global_batch": count, "prompt_len_min": low,
                   "prompt_len_max": high, "seq_len": CONTEXT_LEN, "prefill_chunk": chunk or 0,
                   "generated_tokens": generated, "prompt_tokens": prompt_tokens, "parallelism": "single GPU"},
        "spread": {"min": round(times[0][1] / times[0][0], 1), "median": round(generated / elapsed, 1),
                   "max": round(times[-1][1] / times[-1][0], 1)},
    }


def run_sweep(args):
    """Further sizes: decode steps over batch sizes and context lengths, prompts of many lengths
    whole and in chunks of 256.  GPT-2 XL's layer sizes with room for 8,192 positions and
    ``--layers`` layers (12 unless given: the cache of 64 sequences of 8,192 tokens through 48 layers
    would be 160 GB); every line is tab-separated text, not the one JSON line of the default run."""
    import torch

    import burn_transformers_amd as bt
    layers = args.layers if args.layers != XL["n_layer"] else 12
    dtype = args.dtype or "bf16"
    config = dict(XL, n_layer=layers, n_positions=8192)
    model = build_model(config, dtype)
    vocab = config["vocab_size"]
    weight_bytes, kv_per_token, _ = model_bytes_and_flops(config, layers, dtype)
    d, m = config["n_embd"], config["n_inner"]
    per_layer = 3 * d * d + d * d + 2 * d * m
    print(f"# GPT-2 XL layer sizes, {layers} layers, 8,192 positions, {dtype}, random weights")
    print("# decode: one token per sequence from a HIP graph, every sequence holding `context` tokens")
    print("kind\tbatch\tcontext\tms_per_step\ttokens_per_s\thbm_fraction")
    for context in (1024, 2048, 4096, 8192) if args.sweep_part in ("all", "decode") else ():
        for batch in (1, 8, 16, 32, 64):
            engine = bt.Engine(model, max_tokens=batch * (context + 64))
            slots = [engine.open() for _ in range(batch)]
            prompts = synthetic_prompts(batch, context - 23, vocab, seed=context + batch)
            for begin in range(0, batch, 4):
                engine.step([(slots[i], prompts[i]) for i in range(begin, min(begin + 4, batch))], want=[[] for _ in range(begin, min(begin + 4, batch))])
            ids = [7] * batch
            for _ in range(8):
                engine.step([(slot, [token]) for slot, token in zip(slots, ids)])
            groups = []
            for _ in range(3):                       # the median of three groups of five steps
                torch.cuda.synchronize()
                started = time.perf_counter()
                for _ in range(5):
                    engine.step([(slot, [token]) for slot, token in zip(slots, ids)])
                torch.cuda.synchronize()
                groups.append((time.perf_counter() - started) / 5)
            seconds = sorted(groups)[1]
            nbytes = weight_bytes + batch * context * kv_per_token
            print(f"decode\t{batch}\t{context}\t{seconds * 1e3:.3f}\t{batch / seconds:.0f}\t{nbytes / seconds / 1e9 / PEAK_HBM_GBS:.3f}", flush=True)
            del engine
    print("# prompts: one sequence, whole (chunk 0) or in chunks; the fraction is of the MFMA peak")
    print("kind\ttokens\tchunk\tms\ttokens_per_s\tmfma_fraction")
    engine = bt.Engine(model, max_tokens=8192 + 64)
    for tokens in (64, 128, 256, 512, 1024, 2048, 4096, 8192) if args.sweep_part in ("all", "prompts") else ():
        for chunk in (0, 256):
            if chunk and tokens <= chunk:
                continue
            prompt = synthetic_prompts(1, tokens, vocab, seed=tokens)[0]
            times = []
            for _ in range(5):
                slot = engine.open()
                torch.cuda.synchronize()
                started = time.perf_counter()
                for begin in range(0, tokens, chunk or tokens):
                    engine.step([(slot, prompt[begin:begin + (chunk or tokens)])])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - started)
                engine.close(slot)
            seconds = sorted(times)[1]
            flops = 2.0 * tokens * layers * per_layer + layers * 2.0 * d * tokens * (tokens + 1) + 2.0 * d * vocab
            print(f"prompt\t{tokens}\t{chunk}\t{seconds * 1e3:.3f}\t{tokens / seconds:.0f}\t{flops / seconds / PEAK_FLOPS[dtype]:.3f}", flush=True)


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=CONTEXT_LEN - PROMPT_LEN - 16 - 1)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (48 for GPT-2 XL)")
    parser.add_argument("--model", choices=sorted(MODELS), default="xl",
                        help="whose layer sizes the default workload runs at: GPT-2 XL, medium or small")
    parser.add_argument("--kernel-batches", default="", help="further batch sizes whose decode kernel classes are timed, e.g. 1,64")
    parser.add_argument("--dtype", choices=["bf16", "fp32"], default=None)
    parser.add_argument("--repetitions", type=int, default=10, help="measured repetitions, each on fresh sequences")
    parser.add_argument("--workload", choices=["xl", "small", "medium", "sweep"], default="xl")
    parser.add_argument("--sweep-part", choices=["all", "decode", "prompts"], default="all",
                        help="which table of --workload sweep to run")
    parser.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    parser.add_argument("--no-kernels", action="store_true", help="skip the classes of kernels on their own")
    parser.add_argument("--no-own", action="store_true", help="skip the prefill on this package's own product kernels")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this library")
        sys.exit(2)
    if args.repetitions < 1:
        parser.error("--repetitions must be at least 1")
    args.kernel_batches = [int(b) for b in args.kernel_batches.split(",") if b]
    if args.layers is None:
        args.layers = XL["n_layer"] if args.workload == "sweep" else MODELS[args.model]["n_layer"]
    if args.workload == "sweep":
        run_sweep(args)
    elif args.workload == "xl":
        args.dtype = args.dtype or "bf16"
        print(json.dumps(run_xl(args)))
    else:
        print(json.dumps(run_generation(args)))


if __name__ == "__main__":
    main()
