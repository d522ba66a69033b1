"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and owns no forward pass, cache or loader: every line of the trace becomes
one call of the engine's step function, the one generation uses.  Input, one JSON object per
line on standard input:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries`` give each request's next tokens and the places among them whose logits are wanted;
``end`` lists requests that are finished after the step (their slot and blocks are given back).
For a step with wanted places the float32 logits [places, vocab] go to ``<out>/<step>.f32`` in
the order of the entries and of ``want``.  After every step a line ``done <step>`` is printed
and flushed.
"""

import json
import os
import sys

import numpy as np


class Replay:
    def __init__(self, engine, out_dir):
        self.engine, self.out_dir = engine, out_dir
        self.slots = {}
        os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record):
        entries, want = [], []
        for entry in record.get("entries", []):
            request = entry["id"]
            if not entry["tokens"]:           # nothing to run for this request in this step
                if entry.get("want"):
                    raise ValueError(f"step {record['step']}: request {request!r} wants logits but brings no token")
                continue
            if request not in self.slots:
                self.slots[request] = self.engine.open()
            entries.append((self.slots[request], entry["tokens"]))
            want.append(list(entry.get("want", [])))
        if entries:
            logits = self.engine.step(entries, want)
            if logits.shape[0] > 0:
                data = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                path = os.path.join(self.out_dir, f"{record['step']}.f32")
                with open(path + ".tmp", "wb") as handle:
                    handle.write(np.ascontiguousarray(data).tobytes())
                os.replace(path + ".tmp", path)
        for request in record.get("end", []):
            slot = self.slots.pop(request, None)
            if slot is not None:
                self.engine.close(slot)

    def run(self, lines, out=sys.stdout):
        for line in lines:
            line = line.strip()
            if not line:
                continue
            record = json.loads(line)
            self.run_step(record)
            print(f"done {record['step']}", file=out, flush=True)


def main(argv=None):
    import argparse
    parser = argparse.ArgumentParser(prog="trace_run", description="Replay a trace of token ids and write logits.")
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to 64)")
    args = parser.parse_args(argv)
    from .. import Engine, load_model
    print(f"[trace_run] loading {args.model} ({args.dtype}); kernels are compiled at their first use",
          file=sys.stderr, flush=True)
    model = load_model(args.model, dtype=args.dtype)
    engine = Engine(model, max_tokens=args.max_tokens)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    Replay(engine, args.out).run(sys.stdin)
    return 0
